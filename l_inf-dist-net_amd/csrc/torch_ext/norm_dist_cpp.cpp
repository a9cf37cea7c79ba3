// PyTorch-ROCm C++ extension `norm_dist_cpp`: the module the reference's model/norm_dist.py imports
// (reference model/norm_dist.cpp:92-100 registers the same seven names with pybind11), as a thin layer over the
// C ABI of libldist_hip.so (include/ldist.h).  Same positional arguments, results written into the caller's
// tensors, nothing returned; a tensor that is not on the GPU or not contiguous raises RuntimeError as the
// reference's TORCH_CHECKs do (model/norm_dist.cpp:3-5), and so does a wrong dtype, a shape the operator cannot
// take, or a failed launch (the reference checks neither).  Calls go to the current stream of the tensors' device.
#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <initializer_list>
#include <string>

#include "ldist.h"

namespace {

struct Named {
    const char* name;
    const torch::Tensor& t;
};

// Validates what every entry point asks of its tensors and pins the device for the duration of the call.
class Call {
public:
    Call(const char* op, std::initializer_list<Named> floats, std::initializer_list<Named> ints = {})
        : op_(op) {
        const auto dev = floats.begin()->t.device();
        for (const Named& a : floats) check(a, torch::kFloat32, dev);
        for (const Named& a : ints) check(a, torch::kInt32, dev);
        guard_.set_device(dev);   // only now: the guard takes GPU devices only
    }
    ldist_stream_t stream() const { return (ldist_stream_t)at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }
    void done(int rc) const {
        TORCH_CHECK(rc == LDIST_OK, op_, " failed: ", ldist_strerror(rc),
                    rc == LDIST_ELAUNCH ? " (hipError_t " + std::to_string(ldist_last_hip_error()) + ")" : std::string());
    }

private:
    void check(const Named& a, torch::ScalarType want, const torch::Device& dev) const {
        TORCH_CHECK(a.t.is_cuda(), op_, ": ", a.name, " must be a CUDA tensor");
        TORCH_CHECK(a.t.is_contiguous(), op_, ": ", a.name, " must be contiguous");
        TORCH_CHECK(a.t.scalar_type() == want, op_, ": ", a.name, " must be ", want == torch::kFloat32 ? "float32" : "int32");
        TORCH_CHECK(a.t.device() == dev, op_, ": ", a.name, " is on another device than the first tensor");
    }
    const char* op_;
    at::hip::OptionalHIPGuardMasqueradingAsCUDA guard_;
};

const float* in(const torch::Tensor& t) { return t.data_ptr<float>(); }
float* out(torch::Tensor& t) { return t.data_ptr<float>(); }

// Dimension extraction as the reference does it (model/norm_dist.cpp:26,37,49,59,71,80,88), with the sizes the
// reference leaves unchecked compared first.
struct Shape {
    int B, CO, CI, HW;
};
Shape forward_shape(const char* op, const torch::Tensor& input, const torch::Tensor& weight, const torch::Tensor& output,
                    int G) {
    TORCH_CHECK(input.dim() == 3 && weight.dim() == 2 && output.dim() == 3, op, ": input (B, CI, HW), weight (CO, CI/G), output (B, CO, HW)");
    TORCH_CHECK(G > 0 && weight.size(1) * G == input.size(1), op, ": weight.size(1) * group must equal input.size(1)");
    TORCH_CHECK(output.size(0) == input.size(0) && output.size(1) == weight.size(0) && output.size(2) == input.size(2),
                op, ": output must be (input.size(0), weight.size(0), input.size(2))");
    return {(int)input.size(0), (int)output.size(1), (int)input.size(1), (int)input.size(2)};
}
void same_shape(const char* op, const torch::Tensor& a, const torch::Tensor& b, const char* what) {
    TORCH_CHECK(a.sizes() == b.sizes(), op, ": ", what, " differ in shape");
}

void norm_dist_forward(torch::Tensor& input, torch::Tensor& weight, torch::Tensor& output, int G, float p) {
    Call c("norm_dist_forward", {{"input", input}, {"weight", weight}, {"output", output}});
    const Shape s = forward_shape("norm_dist_forward", input, weight, output, G);
    c.done(ldist_norm_dist_forward(in(input), in(weight), s.B, s.CO, s.CI, G, s.HW, out(output), p, c.stream()));
}

void norm_dist_backward_input(torch::Tensor& grad_output, torch::Tensor& input, torch::Tensor& weight,
                              torch::Tensor& output, torch::Tensor& grad_input, int G, float p) {
    Call c("norm_dist_backward_input", {{"grad_output", grad_output}, {"input", input}, {"weight", weight},
                                        {"output", output}, {"grad_input", grad_input}});
    const Shape s = forward_shape("norm_dist_backward_input", input, weight, output, G);
    same_shape("norm_dist_backward_input", grad_output, output, "grad_output and output");
    same_shape("norm_dist_backward_input", grad_input, input, "grad_input and input");
    c.done(ldist_norm_dist_backward_input(in(grad_output), in(input), in(weight), in(output), s.B, s.CO, s.CI, G, s.HW,
                                          out(grad_input), p, c.stream()));
}

void norm_dist_backward_weight(torch::Tensor& grad_output, torch::Tensor& input, torch::Tensor& weight,
                               torch::Tensor& output, torch::Tensor& grad_weight, int G, float p) {
    Call c("norm_dist_backward_weight", {{"grad_output", grad_output}, {"input", input}, {"weight", weight},
                                         {"output", output}, {"grad_weight", grad_weight}});
    const Shape s = forward_shape("norm_dist_backward_weight", input, weight, output, G);
    same_shape("norm_dist_backward_weight", grad_output, output, "grad_output and output");
    same_shape("norm_dist_backward_weight", grad_weight, weight, "grad_weight and weight");
    c.done(ldist_norm_dist_backward_weight(in(grad_output), in(input), in(weight), in(output), s.B, s.CO, s.CI, G, s.HW,
                                           out(grad_weight), p, c.stream()));
}

void inf_dist_forward(torch::Tensor& input, torch::Tensor& weight, torch::Tensor& output, torch::Tensor& pos, int G) {
    Call c("inf_dist_forward", {{"input", input}, {"weight", weight}, {"output", output}}, {{"pos", pos}});
    const Shape s = forward_shape("inf_dist_forward", input, weight, output, G);
    same_shape("inf_dist_forward", pos, output, "pos and output");
    c.done(ldist_inf_dist_forward(in(input), in(weight), s.B, s.CO, s.CI, G, s.HW, out(output), pos.data_ptr<int32_t>(),
                                  c.stream()));
}

void inf_dist_bound_forward(torch::Tensor& input_lower, torch::Tensor& input_upper, torch::Tensor& weight,
                            torch::Tensor& output_lower, torch::Tensor& output_upper, int G) {
    Call c("inf_dist_bound_forward", {{"input_lower", input_lower}, {"input_upper", input_upper}, {"weight", weight},
                                      {"output_lower", output_lower}, {"output_upper", output_upper}});
    const Shape s = forward_shape("inf_dist_bound_forward", input_lower, weight, output_lower, G);
    same_shape("inf_dist_bound_forward", input_upper, input_lower, "input_upper and input_lower");
    same_shape("inf_dist_bound_forward", output_upper, output_lower, "output_upper and output_lower");
    c.done(ldist_inf_dist_bound_forward(in(input_lower), in(input_upper), in(weight), s.B, s.CO, s.CI, G, s.HW,
                                        out(output_lower), out(output_upper), c.stream()));
}

// The scatter gradients: sizes come from grad_output and the gradient buffer (model/norm_dist.cpp:79-80,87-88); the
// buffers hold what the sums are added to (the reference's caller zero-fills them, model/norm_dist.py:34,37).
void inf_dist_backward_input(torch::Tensor& grad_output, torch::Tensor& pos, torch::Tensor& grad_input, int G) {
    Call c("inf_dist_backward_input", {{"grad_output", grad_output}, {"grad_input", grad_input}}, {{"pos", pos}});
    TORCH_CHECK(grad_output.dim() == 3 && grad_input.dim() == 3 && grad_input.size(0) == grad_output.size(0) &&
                    grad_input.size(2) == grad_output.size(2),
                "inf_dist_backward_input: grad_output (B, CO, HW), grad_input (B, CI, HW)");
    same_shape("inf_dist_backward_input", pos, grad_output, "pos and grad_output");
    c.done(ldist_inf_dist_backward_input(in(grad_output), pos.data_ptr<int32_t>(), (int)grad_output.size(0),
                                         (int)grad_output.size(1), (int)grad_input.size(1), G, (int)grad_output.size(2),
                                         out(grad_input), c.stream()));
}

void inf_dist_backward_weight(torch::Tensor& grad_output, torch::Tensor& pos, torch::Tensor& grad_weight, int G) {
    Call c("inf_dist_backward_weight", {{"grad_output", grad_output}, {"grad_weight", grad_weight}}, {{"pos", pos}});
    TORCH_CHECK(grad_output.dim() == 3 && grad_weight.dim() == 2 && grad_weight.size(0) == grad_output.size(1),
                "inf_dist_backward_weight: grad_output (B, CO, HW), grad_weight (CO, CI/G)");
    same_shape("inf_dist_backward_weight", pos, grad_output, "pos and grad_output");
    c.done(ldist_inf_dist_backward_weight(in(grad_output), pos.data_ptr<int32_t>(), (int)grad_output.size(0),
                                          (int)grad_output.size(1), (int)grad_weight.size(1) * G, G,
                                          (int)grad_output.size(2), out(grad_weight), c.stream()));
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "L_p / L_inf distance-neuron operators for MI355X (gfx950) behind the reference's norm_dist_cpp names";
    m.def("norm_dist_forward", &norm_dist_forward);
    m.def("norm_dist_backward_input", &norm_dist_backward_input);
    m.def("norm_dist_backward_weight", &norm_dist_backward_weight);
    m.def("inf_dist_forward", &inf_dist_forward);
    m.def("inf_dist_bound_forward", &inf_dist_bound_forward);
    m.def("inf_dist_backward_input", &inf_dist_backward_input);
    m.def("inf_dist_backward_weight", &inf_dist_backward_weight);
}
