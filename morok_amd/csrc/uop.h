// Linearized-UOp kernel as it reaches Renderer::render: placeholder, defined with the renderer.
#pragma once
namespace mrk {
struct LinearKernel {};
}  // namespace mrk
