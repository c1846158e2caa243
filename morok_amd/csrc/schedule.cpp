#include "schedule.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <functional>

#include "error.h"

namespace mrk {

// ============================================================================ tensor cores
namespace {

std::vector<TcOpt> opts_from(const char* s) {  // "l0 l0 l0 l0 u1 u1 l1 l1"
    std::vector<TcOpt> v;
    for (const char* p = s; *p; p++)
        if (*p == 'l' || *p == 'u') v.push_back(TcOpt{*p, p[1] - '0'});
    return v;
}
std::vector<SwizzleAxis> sw(std::initializer_list<const char*> items) {
    std::vector<SwizzleAxis> v;
    for (const char* it : items) v.push_back(SwizzleAxis{it[0], it[1] - '0'});
    return v;
}

// renderer.rs:538-547
TensorCore cdna_161616(Scalar in, Scalar out) {
    TensorCore t;
    t.dims = {16, 16, 16};
    t.threads = 64;
    t.elements_per_thread = {4, 4, 4};
    t.dtype_in = in;
    t.dtype_out = out;
    t.opts = opts_from("l0 l0 l0 l0 u1 u1 l1 l1");
    t.swizzle[0] = {sw({"u0", "u1", "l4", "l5", "r2", "r3"}), sw({"r0", "r1"}), sw({"l0", "l1", "l2", "l3"})};
    t.swizzle[1] = {sw({"l0", "l1", "l2", "l3", "r2", "r3"}), sw({"r0", "r1"}), sw({"l4", "l5", "u0", "u1"})};
    return t;
}
// renderer.rs:549-558
TensorCore cdna_161632(Scalar in, Scalar out) {
    TensorCore t;
    t.dims = {16, 16, 32};
    t.threads = 64;
    t.elements_per_thread = {8, 8, 4};
    t.dtype_in = in;
    t.dtype_out = out;
    t.opts = opts_from("l0 l0 l0 l0 u1 u1 l1 l1");
    t.swizzle[0] = {sw({"u0", "u1", "l4", "l5", "r3", "r4"}), sw({"r0", "r1"}), sw({"l0", "l1", "l2", "l3", "r2"})};
    t.swizzle[1] = {sw({"l0", "l1", "l2", "l3", "r3", "r4"}), sw({"r0", "r1"}), sw({"l4", "l5", "u0", "u1", "r2"})};
    return t;
}

// Not in the reference's tables: the 32x32x16 shape of gfx950, the one its matrix pipes sustain
// the highest rate with (register-only streams: 1.70 PFLOP/s against 1.45 for 16x16x32, whose
// instructions move a third more operand bytes per flop).  Lane l holds row / column l % 32 and the
// 8 consecutive k of group l / 32 of A and B; accumulator register e of lane l is
// C[8 * (e / 4) + 4 * (l / 32) + e % 4][l % 32].
TensorCore cdna4_323216(Scalar in, Scalar out) {
    TensorCore t;
    t.dims = {32, 32, 16};
    t.threads = 64;
    t.elements_per_thread = {8, 8, 16};
    t.dtype_in = in;
    t.dtype_out = out;
    t.opts = opts_from("l0 l0 l0 l0 l0 u1 u1 l1 u1 u1");
    t.swizzle[0] = {sw({"u0", "u1", "l5", "u2", "u3", "r3"}), sw({"r0", "r1", "r2", "l0"}), sw({"l1", "l2", "l3", "l4"})};
    t.swizzle[1] = {sw({"l0", "l1", "l2", "l3", "l4", "r3"}), sw({"r0", "r1", "r2", "u0"}), sw({"l5", "u1", "u2", "u3"})};
    return t;
}

const char* tc_dtype_name(Scalar s) {  // tc.rs:677-688
    switch (s) {
        case Scalar::Float16: return "half";
        case Scalar::BFloat16: return "bfloat";
        case Scalar::Float32: return "float";
        case Scalar::Float64: return "double";
        default: return "unknown";
    }
}

// logical axis of every l_i / u_i produced by the opts: (axis 0 = N, 1 = M; bit within axis).
// Each opt splits its axis by 2 and the new range becomes the low part, so successive
// splits of one axis take bits 0, 1, 2, ...
struct Logical {
    int axis;  // 0 N, 1 M, 2 K
    int bit;
};
void logical_axes(const TensorCore& tc, std::vector<Logical>* locals, std::vector<Logical>* upcasts) {
    int next_bit[2] = {0, 0};
    for (const TcOpt& o : tc.opts) {
        Logical l{o.axis, next_bit[o.axis]++};
        (o.kind == 'l' ? locals : upcasts)->push_back(l);
    }
}
Logical resolve(const SwizzleAxis& a, const std::vector<Logical>& locals, const std::vector<Logical>& upcasts) {
    if (a.kind == 'l') return locals[a.idx];
    if (a.kind == 'u') return upcasts[a.idx];
    return Logical{2, a.idx};
}

}  // namespace

std::vector<TensorCore> cdna4_tensor_cores() {  // renderer.rs:724-733, same order
    return {
        cdna_161632(Scalar::Fp8E5M2, Scalar::Float32),
        cdna_161632(Scalar::Fp8E4M3, Scalar::Float32),
        cdna_161632(Scalar::Float16, Scalar::Float32),
        cdna_161632(Scalar::BFloat16, Scalar::Float32),
        cdna_161616(Scalar::Float16, Scalar::Float32),
        cdna_161616(Scalar::BFloat16, Scalar::Float32),
        // additions for gfx950, behind the reference's entries so that selection by dtype is unchanged
        cdna4_323216(Scalar::Float16, Scalar::Float32),
        cdna4_323216(Scalar::BFloat16, Scalar::Float32),
    };
}

RendererCaps amd_cdna4_caps() {
    RendererCaps c;
    c.device = "AMD_CDNA4";
    c.has_local = true;
    c.has_shared = true;
    c.has_threads = false;
    c.shared_max = 163840;
    c.global_max = {2147483647, 65535, 65535};
    c.local_max = 1024;
    c.upcast_max = 8;
    c.tensor_cores = cdna4_tensor_cores();
    return c;
}

int select_tensor_core(const std::vector<TensorCore>& tcs, Scalar in0, Scalar in1, Scalar acc) {
    for (size_t i = 0; i < tcs.size(); i++)
        if (tcs[i].dtype_in == in0 && tcs[i].dtype_in == in1 && tcs[i].dtype_out == acc) return static_cast<int>(i);
    return -1;
}

std::string wmma_name(const TensorCore& tc) {
    return "WMMA_" + std::to_string(tc.dims[0]) + "_" + std::to_string(tc.dims[1]) + "_" + std::to_string(tc.dims[2]) +
           "_" + tc_dtype_name(tc.dtype_in) + "_" + tc_dtype_name(tc.dtype_out);
}

void tc_operand_element(const TensorCore& tc, int operand, int lane, int elem, int* mn, int* k) {
    std::vector<Logical> locals, upcasts;
    logical_axes(tc, &locals, &upcasts);
    const auto& s = tc.swizzle[operand];
    const int relevant = operand == 0 ? 1 : 0;  // A depends on M, B on N
    int out_mn = 0, out_k = 0;
    auto apply = [&](const Logical& l) {
        if (l.axis == 2) out_k |= 1 << l.bit;
        else if (l.axis == relevant) out_mn |= 1 << l.bit;
    };
    // lane bit p <- logical axis at local position p of the operand's view
    for (size_t p = 0; p < s[0].size(); p++)
        if (lane & (1 << p)) apply(resolve(s[0][p], locals, upcasts));
    // element bits: the upcast positions, then the reduce positions, skipping axes the operand
    // does not depend on (those are broadcast in its view)
    int ebit = 0;
    for (int part = 1; part <= 2; part++)
        for (const SwizzleAxis& a : s[part]) {
            Logical l = resolve(a, locals, upcasts);
            if (l.axis != 2 && l.axis != relevant) continue;
            if (elem & (1 << ebit)) apply(l);
            ebit++;
        }
    *mn = out_mn;
    *k = out_k;
}

void tc_acc_element(const TensorCore& tc, int lane, int elem, int* m, int* n) {
    std::vector<Logical> locals, upcasts;
    logical_axes(tc, &locals, &upcasts);
    int om = 0, on = 0;
    for (size_t p = 0; p < locals.size(); p++)
        if (lane & (1 << p)) (locals[p].axis == 0 ? on : om) |= 1 << locals[p].bit;
    for (size_t p = 0; p < upcasts.size(); p++)
        if (elem & (1 << p)) (upcasts[p].axis == 0 ? on : om) |= 1 << upcasts[p].bit;
    *m = om;
    *n = on;
}

// ============================================================================ gpudims
size_t find_smallest_divisor(size_t n) {
    if (n <= 1) return 1;
    size_t lim = static_cast<size_t>(std::ceil(std::sqrt(static_cast<double>(n))));
    for (size_t d = 2; d <= lim; d++)
        if (n % d == 0) return d;
    return 1;  // prime (the reference reports primes, 2 and 3 included via the sqrt bound, as "no divisor")
}

bool group_dims(const std::vector<size_t>& dims, const std::vector<size_t>& max_sizes, std::vector<size_t>* out) {
    std::vector<size_t> r = dims;
    auto fits = [&]() {
        if (r.size() > max_sizes.size()) return false;
        for (size_t i = 0; i < r.size(); i++)
            if (r[i] > max_sizes[i]) return false;
        return true;
    };
    while (!fits()) {
        bool grouped = false;
        size_t lim = std::min(max_sizes.size(), r.size() ? r.size() - 1 : 0);
        for (size_t i = 0; i < lim; i++) {
            if (i + 1 >= r.size()) break;
            unsigned __int128 prod = static_cast<unsigned __int128>(r[i]) * r[i + 1];
            if (prod <= max_sizes[i]) {
                r[i] = static_cast<size_t>(prod);
                r.erase(r.begin() + static_cast<long>(i) + 1);
                grouped = true;
                break;
            }
        }
        if (!grouped) return false;
    }
    *out = r;
    return true;
}

std::vector<size_t> split_dims(const std::vector<size_t>& dims, const std::vector<size_t>& max_sizes) {
    std::vector<size_t> r = dims;
    while (r.size() < 3) r.push_back(1);
    for (size_t i = 0; i < r.size(); i++) {
        size_t mx = i < max_sizes.size() ? max_sizes[i] : static_cast<size_t>(-1);
        while (r[i] > mx) {
            size_t d = find_smallest_divisor(r[i]);
            if (d == 1) break;
            size_t next = (i + 1) % r.size();
            r[i] /= d;
            r[next] *= d;
        }
    }
    while (r.size() > 1 && r.back() == 1) r.pop_back();
    return r;
}

std::vector<size_t> limit_dims(const std::vector<size_t>& dims, const std::vector<size_t>& max_sizes) {
    std::vector<size_t> g;
    if (group_dims(dims, max_sizes, &g)) return g;
    return split_dims(dims, max_sizes);
}

bool get_contraction(const std::vector<size_t>& original, const std::vector<size_t>& limited,
                     std::vector<std::vector<size_t>>* out) {
    out->clear();
    if (original.empty() && limited.empty()) return true;
    if (limited.empty()) return false;
    std::vector<size_t> acc_old, acc_new;
    size_t a = 1;
    for (size_t x : original) acc_old.push_back(a *= x);
    a = 1;
    for (size_t x : limited) acc_new.push_back(a *= x);
    std::vector<size_t> split;
    for (size_t acc : acc_new) {
        if (acc == 1) {
            split.push_back(0);
            continue;
        }
        auto it = std::find(acc_old.begin(), acc_old.end(), acc);
        if (it == acc_old.end()) return false;
        split.push_back(static_cast<size_t>(it - acc_old.begin()) + 1);
    }
    size_t prev = 0;
    for (size_t i = 0; i < split.size(); i++) {
        std::vector<size_t> g;
        size_t hi = (i + 1 == split.size()) ? original.size() : split[i];
        for (size_t j = prev; j < hi; j++) g.push_back(j);
        out->push_back(g);
        if (i + 1 != split.size()) prev = split[i];
    }
    return true;
}

GroupedDims get_grouped_dims(const std::vector<size_t>& dims, const std::vector<size_t>* max_sizes, DimOrder order) {
    GroupedDims g;
    g.original = dims;
    g.order = order;
    std::vector<size_t> d = dims;
    if (order == DimOrder::kReverseDims) std::reverse(d.begin(), d.end());
    g.launch = max_sizes ? limit_dims(d, *max_sizes) : d;
    return g;
}

namespace {
// How the launch extents relate to the dims they were made from: untouched, grouped (with the
// contraction), or split / reshaped (flatten and unflatten).
enum class DimRelation { kSame, kGrouped, kFlat };
DimRelation relate(const std::vector<size_t>& d, const std::vector<size_t>& launch, std::vector<std::vector<size_t>>* contraction) {
    if (launch == d) return DimRelation::kSame;
    if (launch.size() < d.size() && get_contraction(d, launch, contraction)) return DimRelation::kGrouped;
    return DimRelation::kFlat;
}
}  // namespace

std::vector<size_t> GroupedDims::map(const std::vector<size_t>& raw) const {
    std::vector<size_t> d = original;
    if (order == DimOrder::kReverseDims) std::reverse(d.begin(), d.end());
    std::vector<size_t> res;
    std::vector<std::vector<size_t>> contraction;
    switch (relate(d, launch, &contraction)) {
        case DimRelation::kSame: res = raw; break;
        case DimRelation::kGrouped:
            // grouped: peel the original dims off each fused index, fastest-varying first
            res.assign(d.size(), 0);
            for (size_t gi = 0; gi < contraction.size(); gi++) {
                size_t cur = raw[gi];
                const auto& grp = contraction[gi];
                for (size_t j = 0; j + 1 < grp.size(); j++) {
                    res[grp[j]] = cur % d[grp[j]];
                    cur /= d[grp[j]];
                }
                if (!grp.empty()) res[grp.back()] = cur;
            }
            break;
        case DimRelation::kFlat: {
            // split or reshaped: flatten the raw indices row-major, unflatten over the original dims
            size_t flat = 0;
            for (size_t i = 0; i < launch.size(); i++) flat = flat * launch[i] + raw[i];
            res.assign(d.size(), 0);
            for (size_t i = d.size(); i-- > 0;) {
                res[i] = flat % d[i];
                flat /= d[i];
            }
            break;
        }
    }
    if (order != DimOrder::kForward) std::reverse(res.begin(), res.end());
    return res;
}

std::vector<uint32_t> GroupedDims::map_nodes(KernelBuilder& b, const std::vector<uint32_t>& raw) const {
    std::vector<size_t> d = original;
    if (order == DimOrder::kReverseDims) std::reverse(d.begin(), d.end());
    std::vector<uint32_t> res;
    std::vector<std::vector<size_t>> contraction;
    auto c = [](size_t v) { return static_cast<int64_t>(v); };
    switch (relate(d, launch, &contraction)) {
        case DimRelation::kSame: res = raw; break;
        case DimRelation::kGrouped:
            res.assign(d.size(), 0);
            for (size_t gi = 0; gi < contraction.size(); gi++) {
                uint32_t cur = raw[gi];
                const auto& grp = contraction[gi];
                for (size_t j = 0; j + 1 < grp.size(); j++) {
                    res[grp[j]] = d[grp[j]] == 1 ? b.ci(0, b.dtype(cur).scalar) : b.imod(cur, c(d[grp[j]]));
                    if (d[grp[j]] != 1) cur = b.idiv(cur, c(d[grp[j]]));
                }
                if (!grp.empty()) res[grp.back()] = cur;
            }
            break;
        case DimRelation::kFlat: {
            uint32_t flat = raw[0];
            for (size_t i = 1; i < launch.size(); i++) flat = b.iadd(b.imul(flat, c(launch[i])), raw[i]);
            res.assign(d.size(), 0);
            for (size_t i = d.size(); i-- > 0;) {
                res[i] = i == 0 ? flat : b.imod(flat, c(d[i]));
                if (i) flat = b.idiv(flat, c(d[i]));
            }
            break;
        }
    }
    if (order != DimOrder::kForward) std::reverse(res.begin(), res.end());
    return res;
}

// ============================================================================ kernel builder
uint32_t KernelBuilder::add(Op op, DType dt, std::vector<uint32_t> src, int64_t arg_i, double arg_f, uint16_t sub,
                            std::string str, std::vector<int64_t> extra) {
    // Common-subexpression elimination for side-effect-free value nodes: an identical node
    // that is still in scope is returned instead of a new one.
    std::string key;
    bool pure = false;
    if (cse_) {
        switch (op) {
            case Op::Const:
            case Op::Binary:
            case Op::Unary:
            case Op::Where:
            case Op::Cast:
            case Op::BitCast:
            case Op::Gep:
            case Op::Index:
            case Op::Vectorize: pure = true; break;
            default: break;
        }
    }
    if (pure) {
        auto put = [&](const void* p, size_t n) { key.append(static_cast<const char*>(p), n); };
        uint16_t head[6] = {static_cast<uint16_t>(op), static_cast<uint16_t>(dt.scalar), dt.vcount,
                            static_cast<uint16_t>(dt.is_ptr), static_cast<uint16_t>(dt.space), sub};
        put(head, sizeof head);
        put(&dt.ptr_size, sizeof dt.ptr_size);
        put(&arg_i, sizeof arg_i);
        put(&arg_f, sizeof arg_f);
        for (uint32_t v : src) put(&v, sizeof v);
        key.push_back('|');
        for (int64_t v : extra) put(&v, sizeof v);
        key.push_back('|');
        key += str;
        auto it = cse_map_.find(key);
        if (it != cse_map_.end()) return it->second;
    }
    // scopes: values defined inside a loop or a conditional are not visible after it closes
    if (cse_ && (op == Op::End || op == Op::EndIf)) {
        size_t closes = op == Op::End ? std::max<size_t>(src.size(), 1) : 1;
        for (size_t i = 0; i < closes && !cse_scopes_.empty(); i++) {
            for (const std::string& k : cse_scopes_.back()) cse_map_.erase(k);
            cse_scopes_.pop_back();
        }
    }
    UOp u;
    u.id = static_cast<uint32_t>(k_.nodes.size()) + 1;
    u.op = op;
    u.dtype = dt;
    u.src = std::move(src);
    u.arg_i = arg_i;
    u.arg_f = arg_f;
    u.sub = sub;
    u.str = std::move(str);
    u.extra = std::move(extra);
    k_.nodes.push_back(std::move(u));
    const uint32_t id = k_.nodes.back().id;
    if (pure) {
        cse_map_.emplace(key, id);
        if (!cse_scopes_.empty()) cse_scopes_.back().push_back(std::move(key));
    }
    if (cse_ && (op == Op::Range || op == Op::If)) cse_scopes_.emplace_back();
    return id;
}

uint32_t KernelBuilder::binary(BinaryOp op, uint32_t a, uint32_t b) {
    DType d = dtype(a);
    switch (op) {
        case BinaryOp::Lt:
        case BinaryOp::Le:
        case BinaryOp::Gt:
        case BinaryOp::Ge:
        case BinaryOp::Eq:
        case BinaryOp::Ne: d = scalar(Scalar::Bool, d.vcount); break;
        default: break;
    }
    return add(Op::Binary, d, {a, b}, 0, 0, static_cast<uint16_t>(op));
}

uint32_t KernelBuilder::iadd(uint32_t a, uint32_t b) {
    const UOp& na = node(a);
    const UOp& nb = node(b);
    if (na.op == Op::Const && na.arg_i == 0) return b;
    if (nb.op == Op::Const && nb.arg_i == 0) return a;
    if (na.op == Op::Const && nb.op == Op::Const) return ci(na.arg_i + nb.arg_i, na.dtype.scalar);
    return binary(BinaryOp::Add, a, b);
}
uint32_t KernelBuilder::imul(uint32_t a, int64_t c) {
    const UOp& na = node(a);
    if (c == 1) return a;
    if (na.op == Op::Const) return ci(na.arg_i * c, na.dtype.scalar);
    if (c == 0) return ci(0, na.dtype.scalar);
    return binary(BinaryOp::Mul, a, ci(c, na.dtype.scalar));
}
uint32_t KernelBuilder::idiv(uint32_t a, int64_t c) {
    const UOp& na = node(a);
    if (c == 1) return a;
    if (na.op == Op::Const) return ci(na.arg_i / c, na.dtype.scalar);
    return binary(BinaryOp::Idiv, a, ci(c, na.dtype.scalar));
}
uint32_t KernelBuilder::imod(uint32_t a, int64_t c) {
    const UOp& na = node(a);
    if (c == 1) return ci(0, na.dtype.scalar);
    if (na.op == Op::Const) return ci(na.arg_i % c, na.dtype.scalar);
    return binary(BinaryOp::Mod, a, ci(c, na.dtype.scalar));
}

std::vector<uint8_t> KernelBuilder::serialize() const {
    std::vector<uint8_t> out;
    auto put = [&](const void* p, size_t n) {
        const uint8_t* b = static_cast<const uint8_t*>(p);
        out.insert(out.end(), b, b + n);
    };
    auto u32 = [&](uint32_t v) { put(&v, 4); };
    auto u16 = [&](uint16_t v) { put(&v, 2); };
    auto u8 = [&](uint8_t v) { put(&v, 1); };
    auto i64 = [&](int64_t v) { put(&v, 8); };
    u32(0x4C4B524Du);
    u32(1);
    u32(static_cast<uint32_t>(k_.nodes.size()));
    for (const UOp& u : k_.nodes) {
        u32(u.id);
        u16(static_cast<uint16_t>(u.op));
        u8(static_cast<uint8_t>(u.dtype.scalar));
        u8(static_cast<uint8_t>((u.dtype.is_ptr ? 1 : 0) | (static_cast<int>(u.dtype.space) << 1)));
        u16(u.dtype.vcount);
        i64(u.dtype.ptr_size);
        u16(static_cast<uint16_t>(u.src.size()));
        for (uint32_t s : u.src) u32(s);
        i64(u.arg_i);
        put(&u.arg_f, 8);
        u16(u.sub);
        u16(static_cast<uint16_t>(u.str.size()));
        put(u.str.data(), u.str.size());
        u16(static_cast<uint16_t>(u.extra.size()));
        for (int64_t e : u.extra) i64(e);
    }
    return out;
}

LinearKernel KernelBuilder::finish() {
    std::vector<uint8_t> bytes = serialize();
    k_.content_hash = fnv1a64(bytes.data(), bytes.size());
    return k_;
}

// ============================================================================ matmul kernels
bool matmul_f32_opts_valid(const MatmulF32Opts& o, int64_t M, int64_t N, int64_t K) {
    if (o.local_x < 1 || o.local_y < 1 || o.local_x * o.local_y > 1024) return false;
    if (o.up_m < 1 || o.up_m > 8 || o.unroll_k < 1 || o.unroll_k > 8) return false;
    if (o.up_m * o.up_n > (o.lds_k ? 64 : 32)) return false;  // accumulator registers per work-item
    if (o.lds_k) {
        const int64_t threads = static_cast<int64_t>(o.local_x) * o.local_y, tile_m = static_cast<int64_t>(o.local_y) * o.up_m,
                      tile_n = static_cast<int64_t>(o.local_x) * o.up_n;
        if (o.lds_k != 8 && o.lds_k != 16 && o.lds_k != 32) return false;
        if (o.up_n != 4 && o.up_n != 8) return false;
        if (o.up_m != 4 && o.up_m != 8) return false;
        if (threads < 64 || threads % 64 || K % o.lds_k) return false;
        // every work-item copies the same whole number of 4-float vectors of each tile
        if ((tile_m * o.lds_k / 4) % threads || (tile_n * o.lds_k / 4) % threads) return false;
        if ((tile_m + 4 + tile_n + 4) * o.lds_k * 4 > 65536) return false;
        return M % tile_m == 0 && N % tile_n == 0 && M > 0 && N > 0 && K > 0;
    }
    if (o.up_n != 1 && o.up_n != 2 && o.up_n != 4) return false;
    return M % (static_cast<int64_t>(o.local_y) * o.up_m) == 0 && N % (static_cast<int64_t>(o.local_x) * o.up_n) == 0 &&
           K % o.unroll_k == 0 && M > 0 && N > 0 && K > 0;
}

// C = A B in f32 with the operand tiles staged through local memory.  Workgroup tile
// (local_y * up_m) x (local_x * up_n), K depth lds_k per stage.  LDS holds A transposed
// ([k][m], pitch tile_m + 4) and B as it lies ([k][n], pitch tile_n + 4): a work-item's up_m rows
// and up_n columns are then whole 16-byte vectors, read once per k and reused up_n / up_m times;
// the 16 lanes of a row of the workgroup read the same A vector (a broadcast) and 256 contiguous
// bytes of B.  Copies: global -> registers (16-byte loads along k for A, along n for B) -> LDS;
// the loads of the next stage are issued before this stage's barrier.
static LinearKernel build_matmul_f32_lds_kernel(int64_t M, int64_t N, int64_t K, const MatmulF32Opts& o) {
    KernelBuilder b;
    b.enable_cse();
    const Scalar f = Scalar::Float32;
    const int un = o.up_n, um = o.up_m, BK = o.lds_k;
    const int threads = o.local_x * o.local_y;
    const int64_t BM = static_cast<int64_t>(o.local_y) * um, BN = static_cast<int64_t>(o.local_x) * un;
    const int64_t PA = BM + 4, PB = BN + 4;
    const int VA = static_cast<int>(BM * BK / 4 / threads), VB = static_cast<int>(BN * BK / 4 / threads);
    uint32_t c = b.param(0, f, M * N), a = b.param(1, f, M * K), bm = b.param(2, f, K * N);
    uint32_t gx = b.special("gidx0", N / BN), gy = b.special("gidx1", M / BM);
    uint32_t lx = b.special("lidx0", o.local_x), ly = b.special("lidx1", o.local_y);
    uint32_t tid = b.iadd(b.imul(ly, o.local_x), lx);
    uint32_t sA = b.define_local(0, f, PA * BK), sB = b.define_local(1, f, PB * BK);
    uint32_t ra = b.define_reg(1, f, VA, 4), rb = b.define_reg(2, f, VB, 4);
    // vector v of a tile: A row v / (BK / 4), k offset 4 * (v % (BK / 4)); B k row v / (BN / 4), column 4 * (v % (BN / 4))
    std::vector<uint32_t> a_row(VA), a_k(VA), b_k(VB), b_col(VB);
    for (int i = 0; i < VA; i++) {
        uint32_t v = b.iadd(tid, b.ci(threads * i));
        a_row[i] = b.idiv(v, BK / 4);
        a_k[i] = b.imul(b.imod(v, BK / 4), 4);
    }
    for (int i = 0; i < VB; i++) {
        uint32_t v = b.iadd(tid, b.ci(threads * i));
        b_k[i] = b.idiv(v, BN / 4);
        b_col[i] = b.imul(b.imod(v, BN / 4), 4);
    }
    auto global_to_regs = [&](uint32_t kbase) {
        for (int i = 0; i < VA; i++) {
            uint32_t row = b.iadd(b.imul(gy, BM), a_row[i]);
            b.store(b.index(ra, b.ci(i)), b.load(b.index(a, b.iadd(b.imul(row, K), b.iadd(kbase, a_k[i]))), 4));
        }
        for (int i = 0; i < VB; i++) {
            uint32_t col = b.iadd(b.imul(gx, BN), b_col[i]);
            b.store(b.index(rb, b.ci(i)), b.load(b.index(bm, b.iadd(b.imul(b.iadd(kbase, b_k[i]), N), col)), 4));
        }
    };
    std::vector<uint32_t> acc(um * un);
    uint32_t zero = b.cf(0.0);
    for (int i = 0; i < um * un; i++) {
        acc[i] = b.index(b.define_reg(3 + i, f, 1), b.ci(0));
        b.store(acc[i], zero);
    }
    const int64_t KT = K / BK;
    global_to_regs(b.ci(0));
    uint32_t r = b.range(KT, 0, AxisType::Reduce);
    for (int i = 0; i < VA; i++) {  // A transposed: element (row, k) to sA[k][row]
        uint32_t v = b.load(b.index(ra, b.ci(i)));
        for (int e = 0; e < 4; e++) b.store(b.index(sA, b.iadd(b.imul(b.iadd(a_k[i], b.ci(e)), PA), a_row[i])), b.gep(v, e));
    }
    for (int i = 0; i < VB; i++) b.store(b.index(sB, b.iadd(b.imul(b_k[i], PB), b_col[i])), b.load(b.index(rb, b.ci(i))));
    uint32_t rn = b.iadd(r, b.ci(1));
    uint32_t knext = b.imul(b.where(b.binary(BinaryOp::Lt, rn, b.ci(KT)), rn, b.ci(KT - 1)), BK);
    global_to_regs(knext);
    b.barrier();
    uint32_t a_base = b.imul(ly, um), b_base = b.imul(lx, un);
    for (int kk = 0; kk < BK; kk++) {
        std::vector<uint32_t> av, bv;
        for (int i = 0; i < um; i += 4) {
            uint32_t v = b.load(b.index(sA, b.iadd(a_base, b.ci(kk * PA + i))), 4);
            for (int e = 0; e < 4; e++) av.push_back(b.gep(v, e));
        }
        for (int j = 0; j < un; j += 4) {
            uint32_t v = b.load(b.index(sB, b.iadd(b_base, b.ci(kk * PB + j))), 4);
            for (int e = 0; e < 4; e++) bv.push_back(b.gep(v, e));
        }
        for (int i = 0; i < um; i++)
            for (int j = 0; j < un; j++) b.store(acc[i * un + j], b.mulacc(av[i], bv[j], b.load(acc[i * un + j])));
    }
    b.barrier();
    b.end({r});
    uint32_t row0 = b.iadd(b.imul(gy, BM), b.imul(ly, um)), col0 = b.iadd(b.imul(gx, BN), b.imul(lx, un));
    for (int i = 0; i < um; i++)
        for (int j = 0; j < un; j += 4) {
            std::vector<uint32_t> vals;
            for (int e = 0; e < 4; e++) vals.push_back(b.load(acc[i * un + j + e]));
            b.store(b.index(c, b.iadd(b.imul(b.iadd(row0, b.ci(i)), N), b.iadd(col0, b.ci(j)))), b.vectorize(vals));
        }
    return b.finish();
}

LinearKernel build_matmul_f32_kernel(int64_t M, int64_t N, int64_t K, const MatmulF32Opts& o) {
    if (o.lds_k) return build_matmul_f32_lds_kernel(M, N, K, o);
    KernelBuilder b;
    const Scalar f = Scalar::Float32;
    const int un = o.up_n, um = o.up_m;
    const int64_t tile_n = static_cast<int64_t>(o.local_x) * un, tile_m = static_cast<int64_t>(o.local_y) * um;
    uint32_t c = b.param(0, f, M * N), a = b.param(1, f, M * K), bm = b.param(2, f, K * N);
    uint32_t gx = b.special("gidx0", N / tile_n), gy = b.special("gidx1", M / tile_m);
    uint32_t lx = b.special("lidx0", o.local_x), ly = b.special("lidx1", o.local_y);
    uint32_t col0 = b.iadd(b.imul(gx, tile_n), b.imul(lx, un));
    uint32_t row0 = b.iadd(b.imul(gy, tile_m), b.imul(ly, um));
    uint32_t acc = b.define_reg(0, f, um * un);
    uint32_t zero = b.cf(0.0);
    for (int i = 0; i < um * un; i++) b.store(b.index(acc, b.ci(i)), zero);
    uint32_t r = b.range(K / o.unroll_k, 0, AxisType::Reduce);
    for (int u = 0; u < o.unroll_k; u++) {
        uint32_t kk = b.iadd(b.imul(r, o.unroll_k), b.ci(u));
        uint32_t bvec = b.load(b.index(bm, b.iadd(b.imul(kk, N), col0)), un);
        for (int i = 0; i < um; i++) {
            uint32_t arow = b.iadd(row0, b.ci(i));
            uint32_t av = b.load(b.index(a, b.iadd(b.imul(arow, K), kk)));
            for (int j = 0; j < un; j++) {
                uint32_t slot = b.index(acc, b.ci(i * un + j));
                b.store(slot, b.mulacc(av, un > 1 ? b.gep(bvec, j) : bvec, b.load(slot)));
            }
        }
    }
    b.end({r});
    for (int i = 0; i < um; i++) {
        uint32_t arow = b.iadd(row0, b.ci(i));
        std::vector<uint32_t> vals;
        for (int j = 0; j < un; j++) vals.push_back(b.load(b.index(acc, b.ci(i * un + j))));
        b.store(b.index(c, b.iadd(b.imul(arow, N), col0)), un > 1 ? b.vectorize(vals) : vals[0]);
    }
    return b.finish();
}

LinearKernel build_matmul_f32_kernel(int64_t M, int64_t N, int64_t K) { return build_matmul_f32_kernel(M, N, K, MatmulF32Opts()); }

int build_wmma_matmul_kernel(const TensorCore& tc, int64_t M, int64_t N, int64_t K, Scalar out, LinearKernel* k) {
    const int tn = tc.dims[0], tm = tc.dims[1], tk = tc.dims[2];
    if (M % tm || N % tn || K % tk)
        return failf(kInvalidArgument, "tensor-core matmul: shape %lldx%lldx%lld is not a multiple of the %dx%dx%d tile (PADTO is not applied here)",
                     (long long)M, (long long)N, (long long)K, tm, tn, tk);
    if (tc.threads != 64) return fail(kInvalidArgument, "tensor-core matmul: only 64-lane tensor cores are lowered");
    // post-TC upcasts (heuristics.rs:787-821): first of [5,4,3,2] that divides the tile count
    auto pick = [](int64_t tiles) {
        for (int u : {5, 4, 3, 2})
            if (tiles % u == 0) return u;
        return 1;
    };
    const int um = pick(M / tm), un = pick(N / tn);
    const int ea = tc.elements_per_thread[0], eb = tc.elements_per_thread[1], ec = tc.elements_per_thread[2];
    KernelBuilder b;
    uint32_t c = b.param(0, out, M * N), a = b.param(1, tc.dtype_in, M * K), bm = b.param(2, tc.dtype_in, K * N);
    uint32_t gx = b.special("gidx0", N / (tn * un)), gy = b.special("gidx1", M / (tm * um));
    uint32_t lane = b.special("lidx0", 64);  // the WARP range of tc.threads lanes (tc.rs:452-456)
    // per-lane operand coordinates from the swizzle tables, as bit gathers of the lane id.
    // coordinates of element 0; further elements differ only in k (checked below).
    auto lane_expr = [&](int operand, bool want_k) -> uint32_t {
        // value(lane) = sum over lane bits p of bit(lane, p) * contribution(p)
        uint32_t acc_id = b.ci(0);
        for (int p = 0; p < 6; p++) {
            int mn, kk, mn0, kk0;
            tc_operand_element(tc, operand, 1 << p, 0, &mn, &kk);
            tc_operand_element(tc, operand, 0, 0, &mn0, &kk0);
            int contrib = want_k ? kk - kk0 : mn - mn0;
            if (!contrib) continue;
            uint32_t bit = b.binary(BinaryOp::And, b.binary(BinaryOp::Shr, lane, b.ci(p)), b.ci(1));
            acc_id = b.iadd(acc_id, b.imul(bit, contrib));
        }
        return acc_id;
    };
    // element e of a lane must advance k by a lane-independent amount and leave m/n alone
    std::vector<int> a_dk(ea), b_dk(eb);
    for (int operand = 0; operand < 2; operand++)
        for (int e = 0; e < (operand ? eb : ea); e++) {
            int mn, kk, mn0, kk0;
            tc_operand_element(tc, operand, 37, e, &mn, &kk);
            tc_operand_element(tc, operand, 37, 0, &mn0, &kk0);
            if (mn != mn0) return fail(kInvalidArgument, "tensor-core matmul: operand elements span rows/columns");
            (operand ? b_dk : a_dk)[e] = kk - kk0;
        }
    bool a_contig = true;
    for (int e = 0; e < ea; e++) a_contig = a_contig && a_dk[e] == e;
    uint32_t a_m = lane_expr(0, false), a_k = lane_expr(0, true);
    uint32_t b_n = lane_expr(1, false), b_k = lane_expr(1, true);
    // accumulator coordinates
    uint32_t c_m = b.ci(0), c_n = b.ci(0);
    for (int p = 0; p < 6; p++) {
        int m, n;
        tc_acc_element(tc, 1 << p, 0, &m, &n);
        uint32_t bit = b.binary(BinaryOp::And, b.binary(BinaryOp::Shr, lane, b.ci(p)), b.ci(1));
        if (m) c_m = b.iadd(c_m, b.imul(bit, m));
        if (n) c_n = b.iadd(c_n, b.imul(bit, n));
    }
    uint32_t acc = b.define_reg(0, tc.dtype_out, um * un, ec);
    {
        std::vector<uint32_t> z(ec, b.cf(0.0, tc.dtype_out));
        uint32_t zv = b.vectorize(z);
        for (int i = 0; i < um * un; i++) b.store(b.index(acc, b.ci(i)), zv);
    }
    const std::string name = wmma_name(tc);
    uint32_t r = b.range(K / tk, 0, AxisType::Reduce);
    uint32_t kbase = b.imul(r, tk);
    std::vector<uint32_t> afrag(um), bfrag(un);
    for (int i = 0; i < um; i++) {
        uint32_t row = b.iadd(b.iadd(b.imul(gy, tm * um), b.ci(i * tm)), a_m);
        uint32_t base = b.iadd(b.imul(row, K), b.iadd(kbase, a_k));
        if (a_contig) {
            afrag[i] = b.load(b.index(a, base), ea);
        } else {
            std::vector<uint32_t> el;
            for (int e = 0; e < ea; e++) el.push_back(b.load(b.index(a, b.iadd(base, b.ci(a_dk[e])))));
            afrag[i] = b.vectorize(el);
        }
    }
    for (int j = 0; j < un; j++) {
        uint32_t col = b.iadd(b.iadd(b.imul(gx, tn * un), b.ci(j * tn)), b_n);
        std::vector<uint32_t> el;
        for (int e = 0; e < eb; e++) {
            uint32_t krow = b.iadd(b.iadd(kbase, b_k), b.ci(b_dk[e]));
            el.push_back(b.load(b.index(bm, b.iadd(b.imul(krow, N), col))));
        }
        bfrag[j] = b.vectorize(el);
    }
    for (int i = 0; i < um; i++)
        for (int j = 0; j < un; j++) {
            uint32_t slot = b.index(acc, b.ci(i * un + j));
            DType cd = KernelBuilder::scalar(tc.dtype_out, ec);
            uint32_t w = b.add(Op::Wmma, cd, {afrag[i], bfrag[j], b.load(slot)}, 0, 0, 0, name);
            b.store(slot, w);
        }
    b.end({r});
    for (int i = 0; i < um; i++)
        for (int j = 0; j < un; j++) {
            uint32_t res = b.load(b.index(acc, b.ci(i * un + j)));
            for (int e = 0; e < ec; e++) {
                int m, n, m0, n0;
                tc_acc_element(tc, 0, e, &m, &n);
                tc_acc_element(tc, 0, 0, &m0, &n0);
                uint32_t row = b.iadd(b.iadd(b.imul(gy, tm * um), b.ci(i * tm + (m - m0))), c_m);
                uint32_t col = b.iadd(b.iadd(b.imul(gx, tn * un), b.ci(j * tn + (n - n0))), c_n);
                uint32_t v = b.gep(res, e);
                if (out != tc.dtype_out) v = b.cast(v, out);
                b.store(b.index(c, b.iadd(b.imul(row, N), col)), v);
            }
        }
    *k = b.finish();
    return kOk;
}

static bool wmma_async_tile(const TensorCore& tc, const WmmaLdsOpts& o, int* bm, int* bn);

bool wmma_lds_tile(const TensorCore& tc, const WmmaLdsOpts& o, int64_t K, int* bm, int* bn, int* bk) {
    if (o.stages == 2 || o.stages == 3) {
        *bk = 64;
        return wmma_async_tile(tc, o, bm, bn);
    }
    const int tn = tc.dims[0], tm = tc.dims[1], tk = tc.dims[2];
    auto pow2_upto = [](int v, int hi) { return v >= 1 && v <= hi && (v & (v - 1)) == 0; };
    if (!pow2_upto(o.waves_m, 8) || !pow2_upto(o.waves_n, 8) || o.waves_m * o.waves_n > 16) return false;
    if (!pow2_upto(o.up_m, 8) || !pow2_upto(o.up_n, 8) || o.up_m * o.up_n > 32) return false;
    int ku = o.unroll_k;
    if (ku == 0) {
        ku = 1;
        while (ku * 2 * tk <= 64 && K % (ku * 2 * tk) == 0) ku *= 2;
    }
    if (!pow2_upto(ku, 8) || ku * tk > 128) return false;
    *bm = o.waves_m * o.up_m * tm;
    *bn = o.waves_n * o.up_n * tn;
    *bk = ku * tk;
    return true;
}

static bool wmma_async_opts_valid(const TensorCore& tc, const WmmaLdsOpts& o, int64_t M, int64_t N, int64_t K);

bool wmma_lds_opts_valid(const TensorCore& tc, const WmmaLdsOpts& o, int64_t M, int64_t N, int64_t K) {
    if (o.stages == 2 || o.stages == 3) return wmma_async_opts_valid(tc, o, M, N, K);
    if (o.stages != 0) return false;
    if (tc.dtype_in != Scalar::BFloat16 && tc.dtype_in != Scalar::Float16) return false;  // 8 elements per 16-byte copy
    int BM, BN, BK;
    if (tc.threads != 64 || tc.dims[0] != 16 || tc.dims[1] != 16 || !wmma_lds_tile(tc, o, K, &BM, &BN, &BK)) return false;
    // extents that the tile does not divide are padded (PADTO); the 16-byte copies still need
    // rows of whole 8-element vectors
    if (M <= 0 || N <= 0 || K <= 0 || N % 8 || K % 8 || BK % 8) return false;
    const int threads = 64 * o.waves_m * o.waves_n;
    // every work-item copies the same whole number of 8-element vectors of each tile
    if ((BM * BK / 8) % threads || (BK * BN / 8) % threads) return false;
    // both tiles (with their padding) in the 160 KB of local memory, two workgroups per CU
    const size_t lds = (static_cast<size_t>(BM) * (BK + 8) + static_cast<size_t>(BK) * (BN + 4)) * 2;
    return lds <= 80 * 1024;
}

// ---- stages = 2: direct global -> local copies, transposing B reads ------------------------
// Layout of one stage.  A tile [BM][64]: rows of 128 bytes, the eight 16-byte pieces of row r
// XOR-swizzled by (r >> 1) & 7, so the 16 rows a fragment read touches at one k lie in 16
// different bank groups.  B tile [64][BN] as in global memory (n contiguous), its 32-byte
// granules (16 columns) XOR-swizzled by k & 3, so the four k rows of a transposing read lie in
// four different granules.  A copy instruction fills 1 KB of contiguous local memory from 64
// per-lane sources; the swizzles are applied on the source side.
static bool wmma_async_tile(const TensorCore& tc, const WmmaLdsOpts& o, int* bm, int* bn) {
    auto pow2_upto = [](int v, int hi) { return v >= 1 && v <= hi && (v & (v - 1)) == 0; };
    const bool t16 = tc.dims[0] == 16 && tc.dims[1] == 16 && tc.dims[2] == 32, t32 = tc.dims[0] == 32 && tc.dims[1] == 32 && tc.dims[2] == 16;
    if (tc.threads != 64 || (!t16 && !t32)) return false;
    if (tc.dtype_in != Scalar::BFloat16 && tc.dtype_in != Scalar::Float16) return false;
    if (!pow2_upto(o.waves_m, 8) || !pow2_upto(o.waves_n, 8) || o.waves_m * o.waves_n > 16) return false;
    if (!pow2_upto(o.up_m, 8) || !pow2_upto(o.up_n, 8)) return false;
    if (o.up_m * o.up_n * tc.elements_per_thread[2] > 256) return false;  // accumulator registers per lane
    if (o.unroll_k != 0 && o.unroll_k != 64 / tc.dims[2]) return false;
    *bm = o.waves_m * o.up_m * tc.dims[1];
    *bn = o.waves_n * o.up_n * tc.dims[0];
    return true;
}

static bool wmma_async_opts_valid(const TensorCore& tc, const WmmaLdsOpts& o, int64_t M, int64_t N, int64_t K) {
    int BM, BN;
    if (!wmma_async_tile(tc, o, &BM, &BN)) return false;
    const int W = o.waves_m * o.waves_n;
    if (M <= 0 || N <= 0 || K <= 0 || M % BM || N % BN || K % 64) return false;
    if (M * K >= (1LL << 31) || K * N >= (1LL << 31) || M * N >= (1LL << 31)) return false;  // 32-bit element indices
    if (BN < 64 || BN > 512) return false;              // whole granule groups per row, at most one row per copy
    if ((BM / 8) % W || (BN / 8) % W) return false;     // every wave copies the same number of 1 KB chunks
    if ((BM / 8 + BN / 8) / W > 32) return false;
    // two stages of the A tile and two (stages = 2) or three (stages = 3) of the B tile in 160 KB
    if ((2 * BM + (o.stages == 3 ? 3 : 2) * BN) * 64 * 2 > 160 * 1024) return false;
    if (o.stages == 3 && (W > 4 || K / 64 <= 2)) return false;  // the three-stage schedule exists for the one-wave-per-SIMD form only
    return true;
}

static int build_wmma_matmul_async_kernel(const TensorCore& tc, int64_t M, int64_t N, int64_t K, Scalar out,
                                          const WmmaLdsOpts& opts, LinearKernel* k) {
    int BM, BN;
    if (!wmma_async_tile(tc, opts, &BM, &BN) || !wmma_async_opts_valid(tc, opts, M, N, K))
        return failf(kInvalidArgument,
                     "tensor-core matmul (direct copies): shape %lldx%lldx%lld does not divide into the workgroup tile with a K step of 64, "
                     "or the tile does not fit two stages of local memory",
                     (long long)M, (long long)N, (long long)K);
    // TD x TD tiles, tk deep; a lane holds row / column l % TD and the 8 consecutive k of group l / TD
    // of each operand; the accumulator of lane l is column l % TD and, in groups of four registers,
    // rows q * (256 / TD) + 4 * (l / TD) + 0..3.  Written out by hand below, checked against the table here.
    const int TD = tc.dims[0], tk = tc.dims[2], KG = 64 / TD, EC = tc.elements_per_thread[2];
    if (tc.elements_per_thread[0] != 8 || tc.elements_per_thread[1] != 8 || EC != TD * TD / 64)
        return fail(kInvalidArgument, "tensor-core matmul (direct copies): unexpected elements per lane");
    for (int l = 0; l < 64; l++) {
        for (int e = 0; e < 8; e++)
            for (int operand = 0; operand < 2; operand++) {
                int mn, kk;
                tc_operand_element(tc, operand, l, e, &mn, &kk);
                if (mn != l % TD || kk != 8 * (l / TD) + e) return fail(kInvalidArgument, "tensor-core matmul (direct copies): unexpected operand layout");
            }
        for (int e = 0; e < EC; e++) {
            int m, n;
            tc_acc_element(tc, l, e, &m, &n);
            if (m != (e / 4) * (256 / TD) + 4 * (l / TD) + e % 4 || n != l % TD)
                return fail(kInvalidArgument, "tensor-core matmul (direct copies): unexpected accumulator layout");
        }
    }
    const int um = opts.up_m, un = opts.up_n, WM = opts.waves_m, WN = opts.waves_n, W = WM * WN;
    const int KS = 64 / tk, HS = KS / 2;  // tensor-core K steps per 64-deep tile, per half of it
    const int64_t KT = K / 64, tiles_m = M / BM, tiles_n = N / BN, T = tiles_m * tiles_n;
    const int A_STAGE = BM * 64, B_STAGE = 64 * BN;  // elements
    // stages = 3: a third stage of the B tile, as in the hand-written kernel.  The copies of tile
    // r + 2 then split over the whole step: its B chunks go out behind the first half's
    // tensor-core instructions (into the stage tile r - 1 left one barrier ago), its A chunks
    // behind the second half's (into the stage tile r has just left), so that the vector-memory
    // path sees a copy every few instructions instead of all of a tile's copies in half a step.
    const int BST = opts.stages == 3 ? 3 : 2;
    const int CA = BM / 8 / W, CB = BN / 8 / W, PRB = BN / 8;
    KernelBuilder b;
    b.enable_cse();
    uint32_t c = b.param(0, out, M * N), a = b.param(1, tc.dtype_in, M * K), bmat = b.param(2, tc.dtype_in, K * N);
    uint32_t bid = b.special("gidx0", T);
    uint32_t lane = b.special("lidx0", 64), wave = b.special("lidx1", W);
    auto bin = [&](BinaryOp op, uint32_t x, uint32_t y) { return b.binary(op, x, y); };
    // workgroup -> tile: ids congruent mod 8 run on one XCD (one L2); give each XCD a contiguous
    // range of tile ids, and walk tile ids in column groups of four tile rows
    uint32_t id = bid;
    if (T >= 8) {
        const int64_t per = T / 8, rem = T % 8;
        uint32_t xcd = b.imod(bid, 8), idx = b.idiv(bid, 8);
        uint32_t extra = rem ? b.where(bin(BinaryOp::Lt, xcd, b.ci(rem)), xcd, b.ci(rem)) : b.ci(0);
        id = b.iadd(b.iadd(b.imul(xcd, per), extra), idx);
    }
    uint32_t tm, tn;
    {
        const int64_t group = 4, group_sz = group * tiles_n;
        uint32_t g = b.idiv(id, group_sz), first_m = b.imul(g, group), in = b.imod(id, group_sz);
        if (tiles_m % group == 0) {
            tm = b.iadd(first_m, b.imod(in, group));
            tn = b.idiv(in, group);
        } else {
            uint32_t left = bin(BinaryOp::Sub, b.ci(tiles_m), first_m);
            uint32_t gm = b.where(bin(BinaryOp::Lt, left, b.ci(group)), left, b.ci(group));
            tm = b.iadd(first_m, bin(BinaryOp::Mod, in, gm));
            tn = bin(BinaryOp::Idiv, in, gm);
        }
    }
    uint32_t wy = b.idiv(wave, WN), wx = b.imod(wave, WN);
    uint32_t lr = b.imod(lane, TD), lgk = b.idiv(lane, TD);  // row / column inside a tile, k group
    uint32_t i16 = b.imod(lane, 16);                         // lane inside its group of 16 (transposing loads)
    uint32_t sA = b.define_local(0, tc.dtype_in, 2LL * A_STAGE), sB = b.define_local(1, tc.dtype_in, (int64_t)BST * B_STAGE);

    // copies: per wave CA chunks of A and CB chunks of B per tile
    std::vector<uint32_t> a_src(CA), a_dst(CA), b_src(CB), b_dst(CB);
    uint32_t a_tile0 = b.imul(tm, (int64_t)BM * K), b_tile0 = b.imul(tn, BN);
    for (int q = 0; q < CA; q++) {
        uint32_t chunk = b.iadd(b.imul(wave, CA), b.ci(q));
        uint32_t row = b.iadd(b.imul(chunk, 8), b.idiv(lane, 8));
        uint32_t sw = bin(BinaryOp::And, bin(BinaryOp::Shr, row, b.ci(1)), b.ci(7));
        uint32_t piece = bin(BinaryOp::Xor, b.imod(lane, 8), sw);
        a_src[q] = b.iadd(a_tile0, b.iadd(b.imul(row, K), b.imul(piece, 8)));
        a_dst[q] = b.imul(chunk, 512);
    }
    for (int q = 0; q < CB; q++) {
        uint32_t chunk = b.iadd(b.imul(wave, CB), b.ci(q));
        uint32_t piece_id = b.iadd(b.imul(chunk, 64), lane);
        uint32_t krow = b.idiv(piece_id, PRB), pp = b.imod(piece_id, PRB);
        uint32_t gran = bin(BinaryOp::Xor, b.idiv(pp, 2), bin(BinaryOp::And, krow, b.ci(3)));
        uint32_t col = b.imul(b.iadd(b.imul(gran, 2), b.imod(pp, 2)), 8);
        b_src[q] = b.iadd(b_tile0, b.iadd(b.imul(krow, N), col));
        b_dst[q] = b.imul(chunk, 512);
    }
    // copy q (of CA + CB) of tile kt into stage `stage`; kt, stage: nodes (uniform)
    // (stage_b: the B stage when it differs from the A stage; 0 = the same)
    auto copy_one = [&](int q, uint32_t kt, uint32_t stage, uint32_t stage_b = 0) {
        if (q < CA) b.async_copy(b.index(a, b.iadd(a_src[q], b.imul(kt, 64))), b.index(sA, b.iadd(a_dst[q], b.imul(stage, A_STAGE))));
        else b.async_copy(b.index(bmat, b.iadd(b_src[q - CA], b.imul(kt, 64 * N))), b.index(sB, b.iadd(b_dst[q - CA], b.imul(stage_b ? stage_b : stage, B_STAGE))));
    };
    auto copy_tile = [&](uint32_t kt, uint32_t stage) {
        for (int q = 0; q < CA + CB; q++) copy_one(q, kt, stage);
    };
    // fragment addresses: lane-dependent base per K step (A) / per column tile (B) + constants.
    // A, K step s: logical 16-byte piece s * KG + lgk of row wy*um*TD + i*TD + lr (swizzle key (lr >> 1) & 7).
    // B, K step s: the 16 lanes of a group address rows k = s*tk + 8*lgk + i16/4 (+4 for the upper
    // half) of granule (wx*un + j) * (TD/16) + (lr / 16), physically XORed with k & 3 = i16 / 4.
    uint32_t a_sw = bin(BinaryOp::And, b.idiv(lr, 2), b.ci(7));
    uint32_t a_row = b.iadd(b.imul(wy, um * TD), lr);
    std::vector<uint32_t> a_base(KS), b_base(un);
    for (int sst = 0; sst < KS; sst++)
        a_base[sst] = b.iadd(b.imul(a_row, 64), b.imul(bin(BinaryOp::Xor, b.iadd(lgk, b.ci(sst * KG)), a_sw), 8));
    uint32_t b_kq = b.idiv(i16, 4);
    for (int j = 0; j < un; j++) {
        uint32_t gl = b.iadd(b.imul(b.iadd(b.imul(wx, un), b.ci(j)), TD / 16), b.idiv(lr, 16));
        uint32_t gran = bin(BinaryOp::Xor, gl, b_kq);
        b_base[j] = b.iadd(b.imul(b.iadd(b.imul(lgk, 8), b_kq), BN), b.iadd(b.imul(gran, 16), b.imul(b.imod(i16, 4), 4)));
    }
    auto read_a = [&](int sst, int i, uint32_t oa) {
        return b.load(b.index(sA, b.iadd(b.iadd(a_base[sst], oa), b.ci(i * TD * 64))), 8);
    };
    auto read_b = [&](int sst, int j, uint32_t ob) {
        uint32_t at = b.iadd(b_base[j], ob);
        uint32_t lo = b.load_tr(b.index(sB, b.iadd(at, b.ci(sst * tk * BN))));
        uint32_t hi = b.load_tr(b.index(sB, b.iadd(at, b.ci((sst * tk + 4) * BN))));
        std::vector<uint32_t> el;
        for (int e = 0; e < 4; e++) el.push_back(b.gep(lo, e));
        for (int e = 0; e < 4; e++) el.push_back(b.gep(hi, e));
        return b.vectorize(el);
    };
    // registers: accumulators (one object per tile) and the fragments of the first half of a
    // tile's K steps, which are read half a step ahead and so live across the loop edge
    std::vector<uint32_t> acc(um * un), fa0(HS * um), fb0(HS * un);
    int reg_id = 1;
    {
        std::vector<uint32_t> z(EC, b.cf(0.0, tc.dtype_out));
        uint32_t zv = b.vectorize(z);
        for (int i = 0; i < um * un; i++) {
            acc[i] = b.index(b.define_reg(reg_id++, tc.dtype_out, 1, EC), b.ci(0));
            b.store(acc[i], zv);
        }
        for (size_t i = 0; i < fa0.size(); i++) fa0[i] = b.index(b.define_reg(reg_id++, tc.dtype_in, 1, 8), b.ci(0));
        for (size_t j = 0; j < fb0.size(); j++) fb0[j] = b.index(b.define_reg(reg_id++, tc.dtype_in, 1, 8), b.ci(0));
    }
    const std::string name = wmma_name(tc);
    const DType cd = KernelBuilder::scalar(tc.dtype_out, EC);
    // the B fragment goes in as the first operand: the tensor core then leaves four consecutive
    // columns of one row in a lane (result rows are written as vectors), same products, same order
    // between(n): emitted behind tensor-core instruction n of the group
    auto mfmas = [&](const std::vector<uint32_t>& af, const std::vector<uint32_t>& bf,  // [h * um + i], [h * un + j]
                     const std::function<void(int)>& between = nullptr) {
        // columns back and forth, so that consecutive tensor-core instructions always share one
        // operand (fewer operand bits toggle; the part's clock under matrix load follows that)
        int n = 0;
        for (int h = 0; h < HS; h++)
            for (int i = 0; i < um; i++)
                for (int jj = 0; jj < un; jj++) {
                    const int j = (i & 1) ? un - 1 - jj : jj;
                    uint32_t slot = acc[i * un + j];
                    b.store(slot, b.add(Op::Wmma, cd, {bf[h * un + j], af[h * um + i], b.load(slot)}, 0, 0, 0, name));
                    if (between) between(n);
                    n++;
                }
    };
    const int cpw = CA + CB;
    copy_tile(b.ci(0), b.ci(0));
    if (KT > 1) copy_tile(b.ci(1), b.ci(1));
    b.wait_async(KT > 1 ? cpw : 0);
    b.barrier();
    for (int h = 0; h < HS; h++) {
        for (int i = 0; i < um; i++) b.store(fa0[h * um + i], read_a(h, i, b.ci(0)));
        for (int j = 0; j < un; j++) b.store(fb0[h * un + j], read_b(h, j, b.ci(0)));
    }
    // One wave per SIMD and an even number of steps: the loop runs two steps per trip, so that the
    // stage of a step is a constant and the fragment reads address it through their immediate
    // offsets instead of one vector addition each.
    const bool two_per_trip = W <= 4 && KT > 2 && KT % 2 == 0;
    uint32_t r_outer = b.range(two_per_trip ? KT / 2 : KT, 0, AxisType::Reduce);
    for (int trip_step = 0; trip_step < (two_per_trip ? 2 : 1); trip_step++) {
        uint32_t r = two_per_trip ? b.iadd(b.imul(r_outer, 2), b.ci(trip_step)) : r_outer;
        uint32_t st = two_per_trip ? b.ci(trip_step) : b.imod(r, 2), sn = two_per_trip ? b.ci(1 - trip_step) : bin(BinaryOp::Sub, b.ci(1), st);
        // B stages of tile r, r + 1 and (three stages) the one tile r + 2 goes to
        uint32_t sb0 = BST == 3 ? b.imod(r, 3) : st, sb1 = BST == 3 ? b.imod(b.iadd(r, b.ci(1)), 3) : sn;
        uint32_t sb2 = BST == 3 ? b.imod(b.iadd(r, b.ci(2)), 3) : st;
        uint32_t oa = b.imul(st, A_STAGE), ob = b.imul(sb0, B_STAGE), na = b.imul(sn, A_STAGE), nb = b.imul(sb1, B_STAGE);
        std::vector<uint32_t> f1a(HS * um), f1b(HS * un), f0a(HS * um), f0b(HS * un);
        const int total = HS * um * un;  // tensor-core instructions per half step
        if (W <= 4 && KT > 2) {
            // One wave per SIMD: nothing fills the gaps a burst of local-memory reads or copies
            // leaves in the wave's instruction stream, so every read and copy goes behind a
            // tensor-core instruction of its own (the renderer keeps written-out tensor-core
            // instructions and their neighbours in this order): the fragments of the second half
            // behind the first half's instructions, the next tile's first-half fragments and the
            // copies of tile r + 2 behind the second half's.  The last two steps copy the last
            // tile again, into stages nobody reads any more, so that the loop has no branch.
            std::vector<std::function<void()>> reads1, reads0;
            // The reads of a group go out in two bursts, behind the first instructions of each half of the group
            // (rows 0 .. um/2-1 and columns 0 .. un/2-1 first, the rest half a group later, still ahead of their
            // first use): the four waves run in step behind a barrier, and one burst of all of a half step's
            // reads queues longer on the LDS than two of half the size (+1 % at 4096^3).
            const bool split_reads = um % 2 == 0 && un % 2 == 0;
            for (int h = 0; h < HS; h++) {
                if (split_reads) {
                    for (int part = 0; part < 2; part++) {
                        for (int i = part * um / 2; i < (part + 1) * um / 2; i++) reads1.push_back([&, h, i] { f1a[h * um + i] = read_a(HS + h, i, oa); });
                        for (int j = part * un / 2; j < (part + 1) * un / 2; j++) reads1.push_back([&, h, j] { f1b[h * un + j] = read_b(HS + h, j, ob); });
                    }
                    for (int part = 0; part < 2; part++) {
                        for (int i = part * um / 2; i < (part + 1) * um / 2; i++) reads0.push_back([&, h, i] { b.store(fa0[h * um + i], read_a(h, i, na)); });
                        for (int j = part * un / 2; j < (part + 1) * un / 2; j++) reads0.push_back([&, h, j] { b.store(fb0[h * un + j], read_b(h, j, nb)); });
                    }
                    continue;
                }
                for (int i = 0; i < um; i++) reads1.push_back([&, h, i] { f1a[h * um + i] = read_a(HS + h, i, oa); });
                for (int j = 0; j < un; j++) reads1.push_back([&, h, j] { f1b[h * un + j] = read_b(HS + h, j, ob); });
                for (int i = 0; i < um; i++) reads0.push_back([&, h, i] { b.store(fa0[h * um + i], read_a(h, i, na)); });
                for (int j = 0; j < un; j++) reads0.push_back([&, h, j] { b.store(fb0[h * un + j], read_b(h, j, nb)); });
            }
            // slot of read closure c when the reads are split over the two halves of the group
            auto slot_of = [&](int c, int nreads) { return c < nreads / 2 ? c : total / 2 + (c - nreads / 2); };
            for (size_t i = 0; i < fa0.size(); i++) f0a[i] = b.load(fa0[i]);
            for (size_t j = 0; j < fb0.size(); j++) f0b[j] = b.load(fb0[j]);
            uint32_t kt2 = bin(BinaryOp::Sub, b.ci(KT - 1), bin(BinaryOp::Max, bin(BinaryOp::Sub, b.ci(KT - 3), r), b.ci(0)));
            size_t done1 = 0;
            int issued_b = 0;
            const int left1 = std::max(1, total - (int)reads1.size());
            const int every1 = std::max(1, left1 / std::max(1, CB));
            mfmas(f0a, f0b, [&](int n) {
                if (split_reads) {
                    const int nr = (int)reads1.size();
                    if (done1 < reads1.size() && n == slot_of((int)done1, nr)) reads1[done1++]();
                    else if (BST == 3) {
                        // three stages: the B chunks of tile r + 2 in the slots without a read, spread evenly
                        const bool read_slot = n < nr / 2 || (n >= total / 2 && n < total / 2 + nr / 2);
                        const int free_index = n < total / 2 ? n - nr / 2 : n - nr;
                        const int spacing = std::max(1, (total - nr) / std::max(1, CB));
                        if (!read_slot && free_index % spacing == 0 && issued_b < CB) copy_one(CA + issued_b++, kt2, st, sb2);
                    }
                    if (n == total - 1) {
                        while (done1 < reads1.size()) reads1[done1++]();
                        while (BST == 3 && issued_b < CB) copy_one(CA + issued_b++, kt2, st, sb2);
                    }
                    return;
                }
                if (done1 < reads1.size()) reads1[done1++]();
                else if (BST == 3 && (n - (int)reads1.size()) % every1 == 0 && issued_b < CB) copy_one(CA + issued_b++, kt2, st, sb2);
                if (n == total - 1) {
                    while (done1 < reads1.size()) reads1[done1++]();
                    while (BST == 3 && issued_b < CB) copy_one(CA + issued_b++, kt2, st, sb2);
                }
            });
            // tile r + 1 has landed in the other stage (with three stages the B chunks of tile r + 2,
            // the newest copies, may still be on their way) and, behind the barrier, nobody reads
            // this A stage any more
            b.wait_async(BST == 3 ? CB : 0);
            b.barrier();
            size_t done0 = 0;
            int issued = 0;
            const int second = BST == 3 ? CA : cpw;  // copies behind the second half: A only, or the whole tile
            const int left = std::max(1, total - (int)reads0.size());
            const int every = std::max(1, left / second);
            mfmas(f1a, f1b, [&](int n) {
                if (split_reads) {
                    const int nr = (int)reads0.size();
                    if (done0 < reads0.size() && n == slot_of((int)done0, nr)) reads0[done0++]();
                    else {
                        // copies in the slots without a read, spread evenly over them
                        const bool read_slot = n < nr / 2 || (n >= total / 2 && n < total / 2 + nr / 2);
                        const int free_index = n < total / 2 ? n - nr / 2 : n - nr;
                        const int spacing = std::max(1, (total - nr) / std::max(1, second));
                        if (!read_slot && free_index % spacing == 0 && issued < second) copy_one(issued++, kt2, st);
                    }
                    if (n == total - 1) {
                        while (done0 < reads0.size()) reads0[done0++]();
                        while (issued < second) copy_one(issued++, kt2, st);
                    }
                    return;
                }
                if (done0 < reads0.size()) reads0[done0++]();
                else if ((n - (int)reads0.size()) % every == 0 && issued < second) copy_one(issued++, kt2, st);
                if (n == total - 1) {
                    while (done0 < reads0.size()) reads0[done0++]();
                    while (issued < second) copy_one(issued++, kt2, st);
                }
            });
        } else {
            for (int h = 0; h < HS; h++) {
                for (int i = 0; i < um; i++) f1a[h * um + i] = read_a(HS + h, i, oa);
                for (int j = 0; j < un; j++) f1b[h * un + j] = read_b(HS + h, j, ob);
            }
            for (size_t i = 0; i < fa0.size(); i++) f0a[i] = b.load(fa0[i]);
            for (size_t j = 0; j < fb0.size(); j++) f0b[j] = b.load(fb0[j]);
            mfmas(f0a, f0b);
            // tile r + 1 has landed in the other stage (issued half a step ago or earlier) and, behind
            // the barrier, nobody reads this stage any more
            b.wait_async(0);
            b.barrier();
            if (KT > 2) {
                uint32_t r2 = b.iadd(r, b.ci(2));
                b.if_(bin(BinaryOp::Lt, r2, b.ci(KT)));
                copy_tile(r2, st);
                b.endif();
            }
            // first half of tile r + 1 (after the last tile: a stale stage, read and never used)
            for (int h = 0; h < HS; h++) {
                for (int i = 0; i < um; i++) b.store(fa0[h * um + i], read_a(h, i, na));
                for (int j = 0; j < un; j++) b.store(fb0[h * un + j], read_b(h, j, nb));
            }
            mfmas(f1a, f1b);
        }
    }
    b.end({r_outer});
    // Result.  A lane holds, per tile, groups of four consecutive columns of one row.  When the result
    // has the operands' 16-bit type the wave first lays its um*TD x un*TD block out in local memory
    // (the tiles' stages are free after one more barrier; the first half of the waves uses the A
    // stages, the second half the B stages; 16-byte pieces XOR-swizzled by the row) and then
    // writes whole 16-byte pieces, contiguous along each row; otherwise every lane stores its
    // groups of four values directly.
    const int RW = um * TD, CW = un * TD, pieces = CW / 8;  // per-wave block, 16-byte pieces per row
    const int QG = EC / 4, qstride = 256 / TD;             // register groups per tile, columns between them
    const bool staged = out == tc.dtype_in && W % 2 == 0 && pieces >= 2 && 64 % pieces == 0 && RW % (64 / pieces) == 0 &&
                        (int64_t)BM * BN / 2 <= 128LL * std::min(BM, BN);
    if (!staged) {
        uint32_t row0 = b.iadd(b.iadd(b.imul(tm, BM), b.imul(wy, RW)), lr);
        uint32_t col0 = b.iadd(b.iadd(b.imul(tn, BN), b.imul(wx, CW)), b.imul(lgk, 4));
        for (int i = 0; i < um; i++)
            for (int j = 0; j < un; j++) {
                uint32_t res = b.load(acc[i * un + j]);
                for (int q = 0; q < QG; q++) {
                    std::vector<uint32_t> el;
                    for (int e = 0; e < 4; e++) {
                        uint32_t v = b.gep(res, 4 * q + e);
                        el.push_back(out != tc.dtype_out ? b.cast(v, out) : v);
                    }
                    uint32_t at = b.iadd(b.imul(b.iadd(row0, b.ci(i * TD)), N), b.iadd(col0, b.ci(j * TD + q * qstride)));
                    b.store(b.index(c, at), b.vectorize(el));
                }
            }
    } else {
        b.barrier();  // every wave has made its last fragment read
        const int mask = std::min(8, pieces) - 1, rows_per_read = 64 / pieces, reads = RW / rows_per_read;
        uint32_t low_half = bin(BinaryOp::Lt, wave, b.ci(W / 2));
        // writes: row i*TD + lr, columns j*TD + q*qstride + 4*lgk .. + 3: piece (j*TD + q*qstride) / 8 + lgk / 2, half lgk % 2
        uint32_t w_sw = bin(BinaryOp::And, lr, b.ci(mask));
        uint32_t w_base = b.iadd(b.imul(lr, CW), b.imul(b.imod(lgk, 2), 4));
        // reads: lane -> row lane / pieces (+ rows_per_read per step), piece lane % pieces
        uint32_t r_row = b.idiv(lane, pieces), r_piece = b.imod(lane, pieces);
        uint32_t g_row0 = b.iadd(b.iadd(b.imul(tm, BM), b.imul(wy, RW)), r_row);
        uint32_t g_col = b.iadd(b.iadd(b.imul(tn, BN), b.imul(wx, CW)), b.imul(r_piece, 8));
        for (int half = 0; half < 2; half++) {
            b.if_(half == 0 ? low_half : b.unary(UnaryOp::Not, low_half));
            uint32_t region = half == 0 ? sA : sB;
            uint32_t base = b.imul(half == 0 ? wave : bin(BinaryOp::Sub, wave, b.ci(W / 2)), RW * CW);
            // A wave reads back only what it staged itself and local memory serves a wave's requests
            // in order, so the rows of tile row i - 1 are read back and stored while tile row i is
            // being converted and staged: the stores start one tile row after the loop ends.
            auto stage_tile_row = [&](int i) {
                for (int j = 0; j < un; j++) {
                    uint32_t res = b.load(acc[i * un + j]);
                    for (int q = 0; q < QG; q++) {
                        std::vector<uint32_t> el;
                        for (int e = 0; e < 4; e++) el.push_back(b.cast(b.gep(res, 4 * q + e), out));
                        // rows i*TD + lr: the swizzle key (row & mask) is lr & mask whatever i
                        uint32_t piece = bin(BinaryOp::Xor, b.iadd(b.idiv(lgk, 2), b.ci((j * TD + q * qstride) / 8)), w_sw);
                        uint32_t at = b.iadd(b.iadd(base, b.iadd(w_base, b.ci(i * TD * CW))), b.imul(piece, 8));
                        b.store(b.index(region, at), b.vectorize(el));
                    }
                }
            };
            auto store_rows = [&](int t) {
                uint32_t row = b.iadd(r_row, b.ci(t * rows_per_read));
                uint32_t piece = bin(BinaryOp::Xor, r_piece, bin(BinaryOp::And, row, b.ci(mask)));
                uint32_t v = b.load(b.index(region, b.iadd(b.iadd(base, b.imul(row, CW)), b.imul(piece, 8))), 8);
                uint32_t at = b.iadd(b.imul(b.iadd(g_row0, b.ci(t * rows_per_read)), N), g_col);
                b.store(b.index(c, at), v);
            };
            const bool by_tile_row = TD % rows_per_read == 0;  // whole read steps per tile row
            int stored = 0;
            for (int i = 0; i < um; i++) {
                stage_tile_row(i);
                if (by_tile_row && i > 0)
                    for (; stored < i * TD / rows_per_read; stored++) store_rows(stored);
            }
            for (; stored < reads; stored++) store_rows(stored);
            b.endif();
        }
    }
    *k = b.finish();
    return kOk;
}

int build_wmma_matmul_lds_kernel(const TensorCore& tc, int64_t M, int64_t N, int64_t K, Scalar out, const WmmaLdsOpts& opts,
                                 LinearKernel* k) {
    if (opts.stages == 2 || opts.stages == 3) return build_wmma_matmul_async_kernel(tc, M, N, K, out, opts, k);
    if (opts.stages != 0)
        return fail(kInvalidArgument, "tensor-core matmul (LDS): stages must be 0 (through registers), 2 (direct copies) or 3 (direct copies, a third stage of the second operand)");
    const int tn = tc.dims[0], tm = tc.dims[1], tk = tc.dims[2];
    if (tc.threads != 64 || tm != 16 || tn != 16) return fail(kInvalidArgument, "tensor-core matmul (LDS): only 64-lane 16x16 tensor cores are lowered");
    int BM, BN, BK;
    if (!wmma_lds_tile(tc, opts, K, &BM, &BN, &BK))
        return fail(kInvalidArgument, "tensor-core matmul (LDS): waves, tiles per wave and K steps must be powers of two within 16 waves, 32 tiles per wave and a 128-deep K tile");
    const int um = opts.up_m, un = opts.up_n, kWavesM = opts.waves_m, kWavesN = opts.waves_n;
    const int ku = BK / tk, threads = 64 * kWavesM * kWavesN;
    if (M <= 0 || N <= 0 || K <= 0 || N % 8 || K % 8)
        return failf(kInvalidArgument, "tensor-core matmul (LDS): shape %lldx%lldx%lld needs N and K to be multiples of 8 (16-byte copies)",
                     (long long)M, (long long)N, (long long)K);
    if (!wmma_lds_opts_valid(tc, opts, M, N, K))
        return fail(kInvalidArgument, "tensor-core matmul (LDS): the tiles do not divide into whole vectors per work-item or do not fit local memory");
    // PADTO (tc.rs:400-432): an extent the workgroup tile does not divide is rounded up; loads
    // beyond the operands are gated to zero and stores beyond the result are skipped
    const bool pad_m = M % BM != 0, pad_n = N % BN != 0, pad_k = K % BK != 0;
    const int64_t Mp = (M + BM - 1) / BM * BM, Np = (N + BN - 1) / BN * BN;
    const int ea = tc.elements_per_thread[0], eb = tc.elements_per_thread[1], ec = tc.elements_per_thread[2];
    if (BK % 8 || ea != eb) return fail(kInvalidArgument, "tensor-core matmul (LDS): unsupported operand shape");
    // both operands: element e of a lane is k + e (consecutive k), same row / column
    for (int operand = 0; operand < 2; operand++)
        for (int e = 0; e < ea; e++) {
            int mn, kk, mn0, kk0;
            tc_operand_element(tc, operand, 37, e, &mn, &kk);
            tc_operand_element(tc, operand, 37, 0, &mn0, &kk0);
            if (mn != mn0 || kk - kk0 != e) return fail(kInvalidArgument, "tensor-core matmul (LDS): lanes must hold consecutive k");
        }
    KernelBuilder b;
    b.enable_cse();
    uint32_t c = b.param(0, out, M * N), a = b.param(1, tc.dtype_in, M * K), bm = b.param(2, tc.dtype_in, K * N);
    uint32_t gx = b.special("gidx0", Np / BN), gy = b.special("gidx1", Mp / BM);
    uint32_t lane = b.special("lidx0", 64), wave = b.special("lidx1", kWavesM * kWavesN);
    uint32_t tid = b.iadd(b.imul(wave, 64), lane);
    uint32_t wy = b.idiv(wave, kWavesN), wx = b.imod(wave, kWavesN);
    auto lane_expr = [&](int operand, bool want_k) -> uint32_t {
        uint32_t v = b.ci(0);
        for (int p = 0; p < 6; p++) {
            int mn, kk, mn0, kk0;
            tc_operand_element(tc, operand, 1 << p, 0, &mn, &kk);
            tc_operand_element(tc, operand, 0, 0, &mn0, &kk0);
            int contrib = want_k ? kk - kk0 : mn - mn0;
            if (!contrib) continue;
            uint32_t bit = b.binary(BinaryOp::And, b.binary(BinaryOp::Shr, lane, b.ci(p)), b.ci(1));
            v = b.iadd(v, b.imul(bit, contrib));
        }
        return v;
    };
    uint32_t a_m = lane_expr(0, false), a_k = lane_expr(0, true);
    uint32_t b_n = lane_expr(1, false), b_k = lane_expr(1, true);
    uint32_t c_m = b.ci(0), c_n = b.ci(0);
    for (int p = 0; p < 6; p++) {
        int m, n;
        tc_acc_element(tc, 1 << p, 0, &m, &n);
        uint32_t bit = b.binary(BinaryOp::And, b.binary(BinaryOp::Shr, lane, b.ci(p)), b.ci(1));
        if (m) c_m = b.iadd(c_m, b.imul(bit, m));
        if (n) c_n = b.iadd(c_n, b.imul(bit, n));
    }
    // local memory.  A tile [BM][P] as it lies in global memory (the pitch of BK + 8 keeps the
    // vector copies 16-byte aligned and moves consecutive rows to different banks); a lane's A
    // fragment is one vector read.  A B fragment is k-strided in global memory, so B is kept
    // with rows k and k+1 interleaved, [BK/2][PB][2]: a work-item copies the same 8 columns
    // of both rows, zips them in registers and writes two 16-byte vectors, and a lane reads
    // its fragment as element pairs, ready for the tensor core without repacking.  (Writing B
    // transposed instead would put the 16 lanes of a copy on two banks.)  PB = BN + 4 puts
    // the four k groups of a fragment, 4 pair-rows apart, 16 banks apart.  A K tile with an
    // odd number of row vectors per work-item has no whole pairs and keeps plain rows,
    // gathered element by element.
    const int a_vecs_per_row = BK / 8, VA = BM * a_vecs_per_row / threads;   // per work-item
    const int b_vecs_per_row = BN / 8, VB = BK * b_vecs_per_row / threads;
    bool pairs = eb % 2 == 0 && VB % 2 == 0;
    for (int p = 0; p < 6 && pairs; p++) {
        int mn, kk, mn0, kk0;
        tc_operand_element(tc, 1, 1 << p, 0, &mn, &kk);
        tc_operand_element(tc, 1, 0, 0, &mn0, &kk0);
        if ((kk - kk0) % 2) pairs = false;
    }
    const int P = BK + 8, PB = BN + 4;
    uint32_t sA = b.define_local(0, tc.dtype_in, (int64_t)BM * P), sB = b.define_local(1, tc.dtype_in, (int64_t)BK * PB);
    // cooperative copies: vectors of 8 elements, every work-item the same number
    if (VA < 1 || VB < 1) return fail(kInvalidArgument, "tensor-core matmul (LDS): K tile too shallow for the workgroup");
    uint32_t ra = b.define_reg(1, tc.dtype_in, VA, 8), rb = b.define_reg(2, tc.dtype_in, VB, 8);
    std::vector<uint32_t> a_row(VA), a_kc(VA), b_krow(VB), b_nc(VB);
    for (int i = 0; i < VA; i++) {
        uint32_t v = b.iadd(tid, b.ci(threads * i));
        a_row[i] = b.idiv(v, a_vecs_per_row);
        a_kc[i] = b.imul(b.imod(v, a_vecs_per_row), 8);
    }
    for (int i = 0; i < VB; i++) {
        if (pairs) {  // vectors 2i and 2i+1 of a work-item: rows 2p and 2p+1, same columns
            uint32_t v = b.iadd(tid, b.ci(threads * (i / 2)));
            b_krow[i] = b.iadd(b.imul(b.idiv(v, b_vecs_per_row), 2), b.ci(i % 2));
            b_nc[i] = b.imul(b.imod(v, b_vecs_per_row), 8);
        } else {
            uint32_t v = b.iadd(tid, b.ci(threads * i));
            b_krow[i] = b.idiv(v, b_vecs_per_row);
            b_nc[i] = b.imul(b.imod(v, b_vecs_per_row), 8);
        }
    }
    auto both = [&](uint32_t x, uint32_t y) { return x == UINT32_MAX ? y : y == UINT32_MAX ? x : b.binary(BinaryOp::And, x, y); };
    auto global_to_regs = [&](uint32_t kbase) {
        for (int i = 0; i < VA; i++) {
            uint32_t row = b.iadd(b.imul(gy, BM), a_row[i]), kcol = b.iadd(kbase, a_kc[i]);
            uint32_t gate = both(pad_m ? b.binary(BinaryOp::Lt, row, b.ci(M)) : UINT32_MAX, pad_k ? b.binary(BinaryOp::Lt, kcol, b.ci(K)) : UINT32_MAX);
            uint32_t at = b.iadd(b.imul(row, K), kcol);
            b.store(b.index(ra, b.ci(i)), b.load(gate == UINT32_MAX ? b.index(a, at) : b.index_gated(a, at, gate), 8));
        }
        for (int i = 0; i < VB; i++) {
            uint32_t col = b.iadd(b.imul(gx, BN), b_nc[i]), krow = b.iadd(kbase, b_krow[i]);
            uint32_t gate = both(pad_n ? b.binary(BinaryOp::Lt, col, b.ci(N)) : UINT32_MAX, pad_k ? b.binary(BinaryOp::Lt, krow, b.ci(K)) : UINT32_MAX);
            uint32_t at = b.iadd(b.imul(krow, N), col);
            b.store(b.index(rb, b.ci(i)), b.load(gate == UINT32_MAX ? b.index(bm, at) : b.index_gated(bm, at, gate), 8));
        }
    };
    // one register object per accumulator tile: as slots of one array the 64 floats become a
    // single register tuple, which the device compiler shuffles around on every K step
    std::vector<uint32_t> acc(um * un);
    {
        std::vector<uint32_t> z(ec, b.cf(0.0, tc.dtype_out));
        uint32_t zv = b.vectorize(z);
        for (int i = 0; i < um * un; i++) {
            acc[i] = b.index(b.define_reg(3 + i, tc.dtype_out, 1, ec), b.ci(0));
            b.store(acc[i], zv);
        }
    }
    const std::string name = wmma_name(tc);
    const int64_t KT = (K + BK - 1) / BK;
    global_to_regs(b.ci(0));
    uint32_t r = b.range(KT, 0, AxisType::Reduce);
    // registers -> local memory
    for (int i = 0; i < VA; i++) b.store(b.index(sA, b.iadd(b.imul(a_row[i], P), a_kc[i])), b.load(b.index(ra, b.ci(i))));
    if (pairs) {
        for (int i = 0; i < VB; i += 2) {
            uint32_t v0 = b.load(b.index(rb, b.ci(i))), v1 = b.load(b.index(rb, b.ci(i + 1)));
            uint32_t prow = b.idiv(b_krow[i], 2);
            for (int h = 0; h < 2; h++) {
                std::vector<uint32_t> zip;
                for (int e = 0; e < 4; e++) {
                    zip.push_back(b.gep(v0, 4 * h + e));
                    zip.push_back(b.gep(v1, 4 * h + e));
                }
                b.store(b.index(sB, b.imul(b.iadd(b.imul(prow, PB), b.iadd(b_nc[i], b.ci(4 * h))), 2)), b.vectorize(zip));
            }
        }
    } else {
        for (int i = 0; i < VB; i++) {  // rows of PB elements are 8-byte aligned: two stores of four
            uint32_t vb = b.load(b.index(rb, b.ci(i)));
            for (int h = 0; h < 2; h++) {
                std::vector<uint32_t> half;
                for (int e = 0; e < 4; e++) half.push_back(b.gep(vb, 4 * h + e));
                b.store(b.index(sB, b.iadd(b.imul(b_krow[i], PB), b.iadd(b_nc[i], b.ci(4 * h)))), b.vectorize(half));
            }
        }
    }
    // the next step's tiles travel while this step computes (the last step reloads its own).
    // The loads are issued ahead of the barrier: the device compiler moves no memory operation
    // across one, and left after it they sink below the tensor-core work, to the end of the
    // step, where the next step waits for them at once
    uint32_t rn = b.iadd(r, b.ci(1));
    uint32_t knext = b.imul(b.where(b.binary(BinaryOp::Lt, rn, b.ci(KT)), rn, b.ci(KT - 1)), BK);
    global_to_regs(knext);
    b.barrier();
    // fragment addresses as one lane-dependent base plus a constant per fragment, so that the
    // constants fold into the instructions' offset fields instead of taking a register each
    uint32_t a_base = b.iadd(b.imul(b.iadd(b.imul(wy, um * tm), a_m), P), a_k);
    uint32_t b_col = b.iadd(b.imul(wx, un * tn), b_n);
    uint32_t b_base = pairs ? b.imul(b.iadd(b.imul(b.idiv(b_k, 2), PB), b_col), 2) : b.iadd(b.imul(b_k, PB), b_col);
    for (int kk = 0; kk < ku; kk++) {
        std::vector<uint32_t> afrag(um), bfrag(un);
        for (int i = 0; i < um; i++)
            afrag[i] = b.load(b.index(sA, b.iadd(a_base, b.ci(i * tm * P + kk * tk))), ea);
        for (int j = 0; j < un; j++) {
            std::vector<uint32_t> el;
            if (pairs) {
                for (int q = 0; q < eb / 2; q++) {
                    uint32_t two = b.load(b.index(sB, b.iadd(b_base, b.ci(((kk * tk / 2 + q) * PB + j * tn) * 2))), 2);
                    el.push_back(b.gep(two, 0));
                    el.push_back(b.gep(two, 1));
                }
            } else {
                for (int e = 0; e < eb; e++)
                    el.push_back(b.load(b.index(sB, b.iadd(b_base, b.ci((kk * tk + e) * PB + j * tn)))));
            }
            bfrag[j] = b.vectorize(el);
        }
        for (int i = 0; i < um; i++)
            for (int j = 0; j < un; j++) {
                uint32_t slot = acc[i * un + j];
                DType cd = KernelBuilder::scalar(tc.dtype_out, ec);
                uint32_t w = b.add(Op::Wmma, cd, {afrag[i], bfrag[j], b.load(slot)}, 0, 0, 0, name);
                b.store(slot, w);
            }
    }
    b.barrier();  // every wave is done with the tiles before the next step overwrites them
    b.end({r});
    for (int i = 0; i < um; i++)
        for (int j = 0; j < un; j++) {
            uint32_t res = b.load(acc[i * un + j]);
            for (int e = 0; e < ec; e++) {
                int m, n, m0, n0;
                tc_acc_element(tc, 0, e, &m, &n);
                tc_acc_element(tc, 0, 0, &m0, &n0);
                uint32_t row = b.iadd(b.iadd(b.iadd(b.imul(gy, BM), b.imul(wy, um * tm)), b.ci(i * tm + (m - m0))), c_m);
                uint32_t col = b.iadd(b.iadd(b.iadd(b.imul(gx, BN), b.imul(wx, un * tn)), b.ci(j * tn + (n - n0))), c_n);
                uint32_t v = b.gep(res, e);
                if (out != tc.dtype_out) v = b.cast(v, out);
                uint32_t inside = both(pad_m ? b.binary(BinaryOp::Lt, row, b.ci(M)) : UINT32_MAX, pad_n ? b.binary(BinaryOp::Lt, col, b.ci(N)) : UINT32_MAX);
                if (inside != UINT32_MAX) b.if_(inside);
                b.store(b.index(c, b.iadd(b.imul(row, N), col)), v);
                if (inside != UINT32_MAX) b.endif();
            }
        }
    *k = b.finish();
    return kOk;
}

}  // namespace mrk
