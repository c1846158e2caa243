#include "device.h"
#include "error.h"
#include "uop.h"
namespace mrk {
namespace {
class HipRenderer final : public Renderer {
  public:
    explicit HipRenderer(int id) : id_(id) {}
    int render(const LinearKernel&, const char*, ProgramSpec*) override { return fail(kRenderError, "renderer not built yet"); }
    int device_id() const override { return id_; }
  private:
    int id_;
};
}  // namespace
std::shared_ptr<Renderer> make_hip_renderer(int device_id) { return std::make_shared<HipRenderer>(device_id); }
}  // namespace mrk
