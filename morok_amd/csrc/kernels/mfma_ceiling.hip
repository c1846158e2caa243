// Calibration kernel: what the matrix pipes of this part sustain when nothing else competes.
// One workgroup of four waves per compute unit; every wave issues the MFMA stream of one
// 256x256 GEMM tile (128 v_mfma_f32_16x16x32_bf16 per 64-deep K step, sixty-four independent
// accumulators, a different set of operand fragments for each of the two 32-deep sub-steps, the
// 8 x 8 tiles walked back and forth as the GEMM kernel walks them) from registers only: no global
// loads, no LDS traffic, no barriers.  The rate
// it reaches is the ceiling a bf16 GEMM kernel is measured against next to the published peak
// (the part lowers its clock under matrix load, so that ceiling sits below the peak).  With
// operands of random bits the 16x16x32 shape sustains about 14 % more than the 32x32x16 shape
// (1.96 against 1.72 PFLOP/s on the same box): it moves less accumulator data per product.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mrk::dev {

typedef __bf16 cal_bf16x8 __attribute__((ext_vector_type(8)));
typedef float cal_f32x4 __attribute__((ext_vector_type(4)));

// operands: 0 = small smooth values (few bits toggle between consecutive instructions), 1 = values
// spread over [-1.7, 1.7) by a hash of (lane, register, element), as the operands of a product of
// random matrices are.  The matrix pipes' power draw, and with it the clock the part sustains,
// depends on how much the operand bits toggle.
// (a template parameter, so that the set-up in front of the loop is straight-line code)
// half: the same stream of v_mfma_f32_16x16x32_f16 on the same values rounded to IEEE half
// precision (eleven significant bits per operand instead of eight).
template <bool random_operands, bool half = false>
__global__ __launch_bounds__(256) void mfma_ceiling_kernel(float* __restrict__ out, int k_steps, float seed) {
    const int lane = threadIdx.x & 63;
    cal_f32x4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][j][e] = 0.0f;
    cal_bf16x8 fa[2][8], fb[2][8];  // [sub-step][tile row / column]
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            if (random_operands) {
                unsigned x = (unsigned)(((threadIdx.x * 8 + i) * 8 + e) * 2 + ks) * 2654435761u + blockIdx.x * 40503u + 12345u;
                x ^= x >> 15;
                x *= 2246822519u;
                x ^= x >> 13;
                unsigned y = x * 3266489917u;
                y ^= y >> 16;
                const float va = ((float)(x >> 8) / 8388608.0f - 1.0f) * 1.7f, vb = ((float)(y >> 8) / 8388608.0f - 1.0f) * 1.7f;
                if (half) {
                    fa[ks][i][e] = __builtin_bit_cast(__bf16, (_Float16)va);
                    fb[ks][i][e] = __builtin_bit_cast(__bf16, (_Float16)vb);
                } else {
                    fa[ks][i][e] = (__bf16)va;
                    fb[ks][i][e] = (__bf16)vb;
                }
            } else {
                fa[ks][i][e] = (__bf16)(seed * (float)(lane + e + i));
                fb[ks][i][e] = (__bf16)(seed * (float)(lane - e - i));
            }
        }
    for (int kt = 0; kt < k_steps; kt++) {
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int i = 0; i < 8; i++)
#pragma unroll
                for (int jj = 0; jj < 8; jj++) {
                    const int j = (i & 1) ? 7 - jj : jj;
                    // written out, with the accumulator tied in place, as in the GEMM kernel
                    if (half) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fb[ks][j]), "v"(fa[ks][i]));
                    else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fb[ks][j]), "v"(fa[ks][i]));
                }
    }
    // the last results must have left the matrix pipe before the vector ALUs read them (the
    // empty statements keep the reads behind the wait)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) asm volatile("" : "+a"(acc[i][j]));
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) s += acc[i][j][e];
    if (s == 12345.678f) out[0] = s;  // never true for the operands above; keeps the work alive
}

}  // namespace mrk::dev

namespace mrk {

int launch_mfma_ceiling(void* stream, void* out, long workgroups, long k_steps, int random_operands) {
    if (workgroups <= 0 || k_steps <= 0 || workgroups > 0x7fffffffL || k_steps > 0x7fffffffL || !out)
        return (int)hipErrorInvalidValue;
    (void)hipGetLastError();
    if (random_operands == 2)
        dev::mfma_ceiling_kernel<true, true><<<(unsigned)workgroups, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<float*>(out), (int)k_steps, 0.001f);
    else if (random_operands)
        dev::mfma_ceiling_kernel<true><<<(unsigned)workgroups, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<float*>(out), (int)k_steps, 0.001f);
    else
        dev::mfma_ceiling_kernel<false><<<(unsigned)workgroups, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<float*>(out), (int)k_steps, 0.001f);
    return (int)hipGetLastError();
}

}  // namespace mrk
