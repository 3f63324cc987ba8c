// PyTorch-ROCm extension module over the C ABI of libnorm_dist_hip.so: the twelve functions the reference's
// extension exports (core/cuda/norm_dist.cpp:191-204: same names, argument orders, void results, tensors passed by
// reference and written in place), the patch-extraction and convolutional entry points, and the library's
// process-wide switches.  Host code only: every kernel lives in the library; this file checks the tensors the way
// the reference's CHECK_INPUT does (core/cuda/norm_dist.cpp:8-12) plus dtype, shape and device agreement, makes the
// tensors' device current, and launches on PyTorch's current stream of that device.
#include <torch/extension.h>

#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <initializer_list>
#include <string>
#include <utility>
#include <vector>

#include "../../../include/norm_dist_hip.h"

namespace {

using torch::Tensor;

struct Arg {
    const char* name;
    const Tensor& t;
    bool is_int;
};

// device + contiguity (the reference's CHECK_INPUT), dtype, one device for all; returns that device's index
int check_all(std::initializer_list<Arg> args) {
    int dev = -1;
    for (const Arg& a : args) {
        TORCH_CHECK(a.t.is_cuda(), a.name, " must be a CUDA tensor");
        TORCH_CHECK(a.t.is_contiguous(), a.name, " must be contiguous");
        const auto want = a.is_int ? torch::kInt32 : torch::kFloat32;
        TORCH_CHECK(a.t.scalar_type() == want, a.name, " must have dtype ", (a.is_int ? "torch.int32" : "torch.float32"),
                    ", got ", a.t.scalar_type());
        if (dev < 0) dev = a.t.get_device();
        TORCH_CHECK(a.t.get_device() == dev, a.name, " is on device ", a.t.get_device(), ", expected ", dev);
    }
    return dev;
}

void raise_on(int rc, const char* what) {
    TORCH_CHECK(rc == 0, what, " failed: ", ndist_status_string(rc), " (status ", rc, ", hip error ",
                ndist_last_hip_error(), ")");
}

// makes `dev` current for the call and hands out PyTorch's current stream on it
struct Launch {
    explicit Launch(int dev) : guard(static_cast<c10::DeviceIndex>(dev)),
                               stream(c10::hip::getCurrentHIPStream(static_cast<c10::DeviceIndex>(dev)).stream()) {}
    c10::hip::HIPGuard guard;
    hipStream_t stream;
};

const float* F(const Tensor& t) { return t.data_ptr<float>(); }
float* FM(Tensor& t) { return t.data_ptr<float>(); }
const int32_t* I(const Tensor& t) { return t.data_ptr<int32_t>(); }
int32_t* IM(Tensor& t) { return t.data_ptr<int32_t>(); }

void need3d(const Tensor& t, const char* name) { TORCH_CHECK(t.dim() == 3, name, " must be [B, C, HW]"); }

// Shape agreement of one operator call (the kernels index every tensor from B, CO, CI, G, HW alone: a tensor of
// another size would be read or written out of bounds).  ins are [B, CI, HW], outs [B, CO, HW], ws [CO, CI / G].
using Named = std::pair<const char*, const Tensor*>;
void agree(int64_t B, int64_t CO, int64_t CI, int64_t G, int64_t HW, std::initializer_list<Named> ins,
           std::initializer_list<Named> outs, std::initializer_list<Named> ws) {
    TORCH_CHECK(G > 0 && CI % G == 0 && CO % G == 0, "groups (", G, ") must divide the ", CI, " input and the ", CO,
                " output features");
    for (const Named& n : ins)
        TORCH_CHECK(n.second->dim() == 3 && n.second->size(0) == B && n.second->size(1) == CI && n.second->size(2) == HW,
                    n.first, " must be [", B, ", ", CI, ", ", HW, "], got ", n.second->sizes());
    for (const Named& n : outs)
        TORCH_CHECK(n.second->dim() == 3 && n.second->size(0) == B && n.second->size(1) == CO && n.second->size(2) == HW,
                    n.first, " must be [", B, ", ", CO, ", ", HW, "], got ", n.second->sizes());
    for (const Named& n : ws)
        TORCH_CHECK(n.second->dim() == 2 && n.second->size(0) == CO && n.second->size(1) * G == CI, n.first, " must be [",
                    CO, ", ", CI / G, "], got ", n.second->sizes());
}
#define NM(t) Named{#t, &t}

// ---- finite p --------------------------------------------------------------------------------------------------
void norm_dist_forward(const Tensor& input, const Tensor& weight, Tensor& output, int G, float p) {
    const int dev = check_all({{"input", input, false}, {"weight", weight, false}, {"output", output, false}});
    need3d(input, "input"); need3d(output, "output");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input)}, {NM(output)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_norm_dist_forward(F(input), F(weight), input.size(0), output.size(1), input.size(1), G, input.size(2),
                                     FM(output), p, L.stream), "norm_dist_forward");
}

void norm_dist_forward_with_max(const Tensor& input, const Tensor& weight, const Tensor& max_output, Tensor& output, int G,
                                float p) {
    const int dev = check_all({{"input", input, false}, {"weight", weight, false}, {"max_output", max_output, false},
                               {"output", output, false}});
    need3d(input, "input"); need3d(output, "output");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input)}, {NM(output), NM(max_output)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_norm_dist_forward_with_max(F(input), F(weight), F(max_output), input.size(0), output.size(1),
                                              input.size(1), G, input.size(2), FM(output), p, L.stream),
             "norm_dist_forward_with_max");
}

void norm_dist_backward_input(const Tensor& grad_output, const Tensor& input, const Tensor& weight, const Tensor& output,
                              Tensor& grad_input, int G, float p) {
    const int dev = check_all({{"grad_output", grad_output, false}, {"input", input, false}, {"weight", weight, false},
                               {"output", output, false}, {"grad_input", grad_input, false}});
    need3d(input, "input"); need3d(output, "output");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input), NM(grad_input)}, {NM(output), NM(grad_output)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_norm_dist_backward_input(F(grad_output), F(input), F(weight), F(output), grad_output.size(0),
                                            output.size(1), input.size(1), G, input.size(2), FM(grad_input), p, L.stream),
             "norm_dist_backward_input");
}

void norm_dist_backward_input_weight(const Tensor& grad_output, const Tensor& input, const Tensor& weight,
                                     const Tensor& output, Tensor& grad_input, Tensor& grad_weight, int G, float p) {
    const int dev = check_all({{"grad_output", grad_output, false}, {"input", input, false}, {"weight", weight, false},
                               {"output", output, false}, {"grad_input", grad_input, false},
                               {"grad_weight", grad_weight, false}});
    need3d(input, "input"); need3d(output, "output");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input), NM(grad_input)}, {NM(output), NM(grad_output)}, {NM(weight), NM(grad_weight)});
    Launch L(dev);
    raise_on(ndist_norm_dist_backward_input_weight(F(grad_output), F(input), F(weight), F(output), grad_output.size(0),
                                                   output.size(1), input.size(1), G, input.size(2), FM(grad_input),
                                                   FM(grad_weight), p, L.stream),
             "norm_dist_backward_input_weight");
}

// no counterpart in the reference: the same without any allocation inside the library
void norm_dist_backward_input_weight_noalloc(const Tensor& grad_output, const Tensor& input, const Tensor& weight,
                                             const Tensor& output, Tensor& grad_input, Tensor& grad_weight, int G,
                                             float p) {
    const int dev = check_all({{"grad_output", grad_output, false}, {"input", input, false}, {"weight", weight, false},
                               {"output", output, false}, {"grad_input", grad_input, false},
                               {"grad_weight", grad_weight, false}});
    need3d(input, "input"); need3d(output, "output");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input), NM(grad_input)}, {NM(output), NM(grad_output)}, {NM(weight), NM(grad_weight)});
    Launch L(dev);
    raise_on(ndist_norm_dist_backward_input_weight_noalloc(F(grad_output), F(input), F(weight), F(output),
                                                           grad_output.size(0), output.size(1), input.size(1), G,
                                                           input.size(2), FM(grad_input), FM(grad_weight), p, L.stream),
             "norm_dist_backward_input_weight_noalloc");
}

// ---- p = infinity ----------------------------------------------------------------------------------------------
void inf_dist_forward(const Tensor& input, const Tensor& weight, Tensor& output, Tensor& pos, int G) {
    const int dev = check_all({{"input", input, false}, {"weight", weight, false}, {"output", output, false},
                               {"pos", pos, true}});
    need3d(input, "input"); need3d(output, "output");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input)}, {NM(output), NM(pos)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_inf_dist_forward(F(input), F(weight), input.size(0), output.size(1), input.size(1), G, input.size(2),
                                    FM(output), IM(pos), L.stream), "inf_dist_forward");
}

void inf_dist_forward_nograd(const Tensor& input, const Tensor& weight, Tensor& output, int G) {
    const int dev = check_all({{"input", input, false}, {"weight", weight, false}, {"output", output, false}});
    need3d(input, "input"); need3d(output, "output");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input)}, {NM(output)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_inf_dist_forward_nograd(F(input), F(weight), input.size(0), output.size(1), input.size(1), G,
                                           input.size(2), FM(output), L.stream), "inf_dist_forward_nograd");
}

void inf_dist_backward_input(const Tensor& grad_output, const Tensor& pos, Tensor& grad_input, int G) {
    const int dev = check_all({{"grad_output", grad_output, false}, {"pos", pos, true}, {"grad_input", grad_input, false}});
    need3d(grad_output, "grad_output"); need3d(grad_input, "grad_input");
    agree(grad_output.size(0), grad_output.size(1), grad_input.size(1), G, grad_output.size(2), {NM(grad_input)}, {NM(grad_output), NM(pos)}, {});
    Launch L(dev);
    raise_on(ndist_inf_dist_backward_input(F(grad_output), I(pos), grad_output.size(0), grad_output.size(1),
                                           grad_input.size(1), G, grad_input.size(2), FM(grad_input), L.stream),
             "inf_dist_backward_input");
}

void inf_dist_backward_input_weight(const Tensor& grad_output, const Tensor& pos, Tensor& grad_input, Tensor& grad_weight,
                                    int G) {
    const int dev = check_all({{"grad_output", grad_output, false}, {"pos", pos, true}, {"grad_input", grad_input, false},
                               {"grad_weight", grad_weight, false}});
    need3d(grad_output, "grad_output");
    TORCH_CHECK(grad_weight.dim() == 2, "grad_weight must be [CO, CI / G]");
    agree(grad_output.size(0), grad_output.size(1), grad_weight.size(1) * G, G, grad_output.size(2), {NM(grad_input)}, {NM(grad_output), NM(pos)}, {NM(grad_weight)});
    Launch L(dev);
    raise_on(ndist_inf_dist_backward_input_weight(F(grad_output), I(pos), grad_output.size(0), grad_output.size(1),
                                                  grad_weight.size(1) * G, G, grad_output.size(2), FM(grad_input),
                                                  FM(grad_weight), L.stream),
             "inf_dist_backward_input_weight");
}

// ---- interval bounds -------------------------------------------------------------------------------------------
void bound_inf_dist_forward(const Tensor& inputL, const Tensor& inputU, const Tensor& weight, Tensor& outputL,
                            Tensor& outputU, Tensor& posL, Tensor& posU, int G) {
    const int dev = check_all({{"inputL", inputL, false}, {"inputU", inputU, false}, {"weight", weight, false},
                               {"outputL", outputL, false}, {"outputU", outputU, false}, {"posL", posL, true},
                               {"posU", posU, true}});
    need3d(inputL, "inputL"); need3d(outputL, "outputL");
    agree(inputL.size(0), outputL.size(1), inputL.size(1), G, inputL.size(2), {NM(inputL), NM(inputU)}, {NM(outputL), NM(outputU), NM(posL), NM(posU)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_bound_inf_dist_forward(F(inputL), F(inputU), F(weight), inputL.size(0), outputL.size(1), inputL.size(1),
                                          G, inputL.size(2), FM(outputL), FM(outputU), IM(posL), IM(posU), L.stream),
             "bound_inf_dist_forward");
}

void bound_inf_dist_forward_nograd(const Tensor& inputL, const Tensor& inputU, const Tensor& weight, Tensor& outputL,
                                   Tensor& outputU, int G) {
    const int dev = check_all({{"inputL", inputL, false}, {"inputU", inputU, false}, {"weight", weight, false},
                               {"outputL", outputL, false}, {"outputU", outputU, false}});
    need3d(inputL, "inputL"); need3d(outputL, "outputL");
    agree(inputL.size(0), outputL.size(1), inputL.size(1), G, inputL.size(2), {NM(inputL), NM(inputU)}, {NM(outputL), NM(outputU)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_bound_inf_dist_forward_nograd(F(inputL), F(inputU), F(weight), inputL.size(0), outputL.size(1),
                                                 inputL.size(1), G, inputL.size(2), FM(outputL), FM(outputU), L.stream),
             "bound_inf_dist_forward_nograd");
}

void bound_inf_dist_backward_input(const Tensor& grad_outputL, const Tensor& grad_outputU, const Tensor& posL,
                                   const Tensor& posU, Tensor& grad_inputL, Tensor& grad_inputU, int G) {
    const int dev = check_all({{"grad_outputL", grad_outputL, false}, {"grad_outputU", grad_outputU, false},
                               {"posL", posL, true}, {"posU", posU, true}, {"grad_inputL", grad_inputL, false},
                               {"grad_inputU", grad_inputU, false}});
    need3d(grad_outputL, "grad_outputL"); need3d(grad_inputL, "grad_inputL");
    agree(grad_outputL.size(0), grad_outputL.size(1), grad_inputL.size(1), G, grad_outputL.size(2), {NM(grad_inputL), NM(grad_inputU)}, {NM(grad_outputL), NM(grad_outputU), NM(posL), NM(posU)}, {});
    Launch L(dev);
    raise_on(ndist_bound_inf_dist_backward_input(F(grad_outputL), F(grad_outputU), I(posL), I(posU), grad_outputL.size(0),
                                                 grad_outputL.size(1), grad_inputL.size(1), G, grad_inputL.size(2),
                                                 FM(grad_inputL), FM(grad_inputU), L.stream),
             "bound_inf_dist_backward_input");
}

void bound_inf_dist_backward_input_weight(const Tensor& grad_outputL, const Tensor& grad_outputU, const Tensor& posL,
                                          const Tensor& posU, Tensor& grad_inputL, Tensor& grad_inputU,
                                          Tensor& grad_weight, int G) {
    const int dev = check_all({{"grad_outputL", grad_outputL, false}, {"grad_outputU", grad_outputU, false},
                               {"posL", posL, true}, {"posU", posU, true}, {"grad_inputL", grad_inputL, false},
                               {"grad_inputU", grad_inputU, false}, {"grad_weight", grad_weight, false}});
    need3d(grad_outputL, "grad_outputL");
    TORCH_CHECK(grad_weight.dim() == 2, "grad_weight must be [CO, CI / G]");
    agree(grad_outputL.size(0), grad_outputL.size(1), grad_weight.size(1) * G, G, grad_outputL.size(2), {NM(grad_inputL), NM(grad_inputU)}, {NM(grad_outputL), NM(grad_outputU), NM(posL), NM(posU)}, {NM(grad_weight)});
    Launch L(dev);
    raise_on(ndist_bound_inf_dist_backward_input_weight(F(grad_outputL), F(grad_outputU), I(posL), I(posU),
                                                        grad_outputL.size(0), grad_outputL.size(1),
                                                        grad_weight.size(1) * G, G, grad_outputL.size(2),
                                                        FM(grad_inputL), FM(grad_inputU), FM(grad_weight), L.stream),
             "bound_inf_dist_backward_input_weight");
}

// a layer's distance and its interval bounds in one call (pre-pass over the weights shared); no counterpart in the
// reference's extension, whose layers make the two calls one after the other (core/modules/norm_dist.py:30-34)
void inf_and_bound_forward_nograd(const Tensor& input, const Tensor& inputL, const Tensor& inputU, const Tensor& weight,
                                  Tensor& output, Tensor& outputL, Tensor& outputU, int G) {
    const int dev = check_all({{"input", input, false}, {"inputL", inputL, false}, {"inputU", inputU, false},
                               {"weight", weight, false}, {"output", output, false}, {"outputL", outputL, false},
                               {"outputU", outputU, false}});
    need3d(input, "input"); need3d(output, "output");
    TORCH_CHECK(input.sizes() == inputL.sizes() && input.sizes() == inputU.sizes(), "input and its bounds must have the same shape");
    TORCH_CHECK(output.sizes() == outputL.sizes() && output.sizes() == outputU.sizes(), "the three outputs must have the same shape");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input), NM(inputL), NM(inputU)}, {NM(output), NM(outputL), NM(outputU)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_inf_and_bound_forward_nograd(F(input), F(inputL), F(inputU), F(weight), input.size(0), output.size(1),
                                                input.size(1), G, input.size(2), FM(output), FM(outputL), FM(outputU),
                                                L.stream), "inf_and_bound_forward_nograd");
}

void inf_and_bound_forward(const Tensor& input, const Tensor& inputL, const Tensor& inputU, const Tensor& weight,
                           Tensor& output, Tensor& pos, Tensor& outputL, Tensor& outputU, Tensor& posL, Tensor& posU, int G) {
    const int dev = check_all({{"input", input, false}, {"inputL", inputL, false}, {"inputU", inputU, false},
                               {"weight", weight, false}, {"output", output, false}, {"pos", pos, true},
                               {"outputL", outputL, false}, {"outputU", outputU, false}, {"posL", posL, true},
                               {"posU", posU, true}});
    need3d(input, "input"); need3d(output, "output");
    TORCH_CHECK(input.sizes() == inputL.sizes() && input.sizes() == inputU.sizes(), "input and its bounds must have the same shape");
    agree(input.size(0), output.size(1), input.size(1), G, input.size(2), {NM(input), NM(inputL), NM(inputU)}, {NM(output), NM(outputL), NM(outputU), NM(pos), NM(posL), NM(posU)}, {NM(weight)});
    Launch L(dev);
    raise_on(ndist_inf_and_bound_forward(F(input), F(inputL), F(inputU), F(weight), input.size(0), output.size(1),
                                         input.size(1), G, input.size(2), FM(output), IM(pos), FM(outputL), FM(outputU),
                                         IM(posL), IM(posU), L.stream), "inf_and_bound_forward");
}

// ---- patch extraction and the convolutional layer without the unfolded tensor ------------------------------------
// geometry: (kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w, stride_h, stride_w)
using Geo = std::vector<int64_t>;
void need_geo(const Geo& g) { TORCH_CHECK(g.size() == 8, "geometry must be (kh, kw, dh, dw, ph, pw, sh, sw)"); }
void need4d(const Tensor& t, const char* name) { TORCH_CHECK(t.dim() == 4, name, " must be [B, C, H, W]"); }
#define GEO8(g) (int)g[0], (int)g[1], (int)g[2], (int)g[3], (int)g[4], (int)g[5], (int)g[6], (int)g[7]
#define IMG4(t) (int)t.size(0), (int)t.size(1), (int)t.size(2), (int)t.size(3)

void unfold_forward(const Tensor& input, Tensor& output, const Geo& geo) {
    need_geo(geo); need4d(input, "input");
    const int dev = check_all({{"input", input, false}, {"output", output, false}});
    Launch L(dev);
    raise_on(ndist_unfold_forward(F(input), IMG4(input), GEO8(geo), FM(output), L.stream), "unfold_forward");
}

void unfold_backward(const Tensor& grad_output, Tensor& grad_input, const Geo& geo) {
    need_geo(geo); need4d(grad_input, "grad_input");
    const int dev = check_all({{"grad_output", grad_output, false}, {"grad_input", grad_input, false}});
    Launch L(dev);
    raise_on(ndist_unfold_backward(F(grad_output), IMG4(grad_input), GEO8(geo), FM(grad_input), L.stream),
             "unfold_backward");
}

void conv_inf_dist_forward_nograd(const Tensor& input, const Tensor& weight, Tensor& output, int G, const Geo& geo) {
    need_geo(geo); need4d(input, "input");
    const int dev = check_all({{"input", input, false}, {"weight", weight, false}, {"output", output, false}});
    Launch L(dev);
    raise_on(ndist_conv_inf_dist_forward_nograd(F(input), F(weight), IMG4(input), (int)weight.size(0), G, GEO8(geo),
                                                FM(output), L.stream), "conv_inf_dist_forward_nograd");
}

void conv_bound_inf_dist_forward_nograd(const Tensor& inputL, const Tensor& inputU, const Tensor& weight, Tensor& outputL,
                                        Tensor& outputU, int G, const Geo& geo) {
    need_geo(geo); need4d(inputL, "inputL");
    const int dev = check_all({{"inputL", inputL, false}, {"inputU", inputU, false}, {"weight", weight, false},
                               {"outputL", outputL, false}, {"outputU", outputU, false}});
    TORCH_CHECK(inputL.sizes() == inputU.sizes() && outputL.sizes() == outputU.sizes(),
                "lower and upper tensors must have the same shape");
    Launch L(dev);
    raise_on(ndist_conv_bound_inf_dist_forward_nograd(F(inputL), F(inputU), F(weight), IMG4(inputL), (int)weight.size(0),
                                                      G, GEO8(geo), FM(outputL), FM(outputU), L.stream),
             "conv_bound_inf_dist_forward_nograd");
}

void conv_inf_dist_forward(const Tensor& input, const Tensor& weight, Tensor& output, Tensor& pos, int G, const Geo& geo) {
    need_geo(geo); need4d(input, "input");
    const int dev = check_all({{"input", input, false}, {"weight", weight, false}, {"output", output, false},
                               {"pos", pos, true}});
    TORCH_CHECK(pos.sizes() == output.sizes(), "pos must have the shape of output");
    Launch L(dev);
    raise_on(ndist_conv_inf_dist_forward(F(input), F(weight), IMG4(input), (int)weight.size(0), G, GEO8(geo), FM(output),
                                         IM(pos), L.stream), "conv_inf_dist_forward");
}

void conv_norm_dist_forward(const Tensor& input, const Tensor& weight, Tensor& output, int G, double p, const Geo& geo) {
    need_geo(geo); need4d(input, "input");
    const int dev = check_all({{"input", input, false}, {"weight", weight, false}, {"output", output, false}});
    Launch L(dev);
    raise_on(ndist_conv_norm_dist_forward(F(input), F(weight), IMG4(input), (int)weight.size(0), G, GEO8(geo), FM(output),
                                          (float)p, L.stream), "conv_norm_dist_forward");
}

void conv_norm_dist_backward_input(const Tensor& grad_output, const Tensor& input, const Tensor& weight,
                                   const Tensor& output, Tensor& grad_input, int G, double p, const Geo& geo) {
    need_geo(geo); need4d(input, "input");
    const int dev = check_all({{"grad_output", grad_output, false}, {"input", input, false}, {"weight", weight, false},
                               {"output", output, false}, {"grad_input", grad_input, false}});
    TORCH_CHECK(grad_output.sizes() == output.sizes() && grad_input.sizes() == input.sizes(),
                "gradients must have the shapes of output and input");
    Launch L(dev);
    raise_on(ndist_conv_norm_dist_backward_input(F(grad_output), F(input), F(weight), F(output), IMG4(input),
                                                 (int)weight.size(0), G, GEO8(geo), FM(grad_input), (float)p, L.stream),
             "conv_norm_dist_backward_input");
}

void conv_norm_dist_backward_input_weight(const Tensor& grad_output, const Tensor& input, const Tensor& weight,
                                          const Tensor& output, Tensor& grad_input, Tensor& grad_weight, int G, double p,
                                          const Geo& geo) {
    need_geo(geo); need4d(input, "input");
    const int dev = check_all({{"grad_output", grad_output, false}, {"input", input, false}, {"weight", weight, false},
                               {"output", output, false}, {"grad_input", grad_input, false},
                               {"grad_weight", grad_weight, false}});
    TORCH_CHECK(grad_output.sizes() == output.sizes() && grad_input.sizes() == input.sizes() &&
                    grad_weight.sizes() == weight.sizes(),
                "gradients must have the shapes of output, input and weight");
    Launch L(dev);
    raise_on(ndist_conv_norm_dist_backward_input_weight(F(grad_output), F(input), F(weight), F(output), IMG4(input),
                                                        (int)weight.size(0), G, GEO8(geo), FM(grad_input),
                                                        FM(grad_weight), (float)p, L.stream),
             "conv_norm_dist_backward_input_weight");
}

void conv_bound_inf_dist_forward(const Tensor& inputL, const Tensor& inputU, const Tensor& weight, Tensor& outputL,
                                 Tensor& outputU, Tensor& posL, Tensor& posU, int G, const Geo& geo) {
    need_geo(geo); need4d(inputL, "inputL");
    const int dev = check_all({{"inputL", inputL, false}, {"inputU", inputU, false}, {"weight", weight, false},
                               {"outputL", outputL, false}, {"outputU", outputU, false}, {"posL", posL, true},
                               {"posU", posU, true}});
    TORCH_CHECK(inputL.sizes() == inputU.sizes() && outputL.sizes() == outputU.sizes() &&
                    posL.sizes() == outputL.sizes() && posU.sizes() == outputL.sizes(),
                "lower and upper tensors must have the same shape");
    Launch L(dev);
    raise_on(ndist_conv_bound_inf_dist_forward(F(inputL), F(inputU), F(weight), IMG4(inputL), (int)weight.size(0), G,
                                               GEO8(geo), FM(outputL), FM(outputU), IM(posL), IM(posU), L.stream),
             "conv_bound_inf_dist_forward");
}

void conv_inf_dist_backward_input(const Tensor& grad_output, const Tensor& pos, Tensor& grad_input, int CO, int G,
                                  const Geo& geo) {
    need_geo(geo); need4d(grad_input, "grad_input");
    const int dev = check_all({{"grad_output", grad_output, false}, {"pos", pos, true}, {"grad_input", grad_input, false}});
    Launch L(dev);
    raise_on(ndist_conv_inf_dist_backward_input(F(grad_output), I(pos), IMG4(grad_input), CO, G, GEO8(geo),
                                                FM(grad_input), L.stream), "conv_inf_dist_backward_input");
}

void conv_inf_dist_backward_input_weight(const Tensor& grad_output, const Tensor& pos, Tensor& grad_input,
                                         Tensor& grad_weight, int G, const Geo& geo) {
    need_geo(geo); need4d(grad_input, "grad_input");
    const int dev = check_all({{"grad_output", grad_output, false}, {"pos", pos, true}, {"grad_input", grad_input, false},
                               {"grad_weight", grad_weight, false}});
    Launch L(dev);
    raise_on(ndist_conv_inf_dist_backward_input_weight(F(grad_output), I(pos), IMG4(grad_input), (int)grad_weight.size(0),
                                                       G, GEO8(geo), FM(grad_input), FM(grad_weight), L.stream),
             "conv_inf_dist_backward_input_weight");
}

void conv_bound_inf_dist_backward_input(const Tensor& grad_outputL, const Tensor& grad_outputU, const Tensor& posL,
                                        const Tensor& posU, Tensor& grad_inputL, Tensor& grad_inputU, int CO, int G,
                                        const Geo& geo) {
    need_geo(geo); need4d(grad_inputL, "grad_inputL");
    const int dev = check_all({{"grad_outputL", grad_outputL, false}, {"grad_outputU", grad_outputU, false},
                               {"posL", posL, true}, {"posU", posU, true}, {"grad_inputL", grad_inputL, false},
                               {"grad_inputU", grad_inputU, false}});
    Launch L(dev);
    raise_on(ndist_conv_bound_inf_dist_backward_input(F(grad_outputL), F(grad_outputU), I(posL), I(posU),
                                                      IMG4(grad_inputL), CO, G, GEO8(geo), FM(grad_inputL),
                                                      FM(grad_inputU), L.stream),
             "conv_bound_inf_dist_backward_input");
}

void conv_bound_inf_dist_backward_input_weight(const Tensor& grad_outputL, const Tensor& grad_outputU, const Tensor& posL,
                                               const Tensor& posU, Tensor& grad_inputL, Tensor& grad_inputU,
                                               Tensor& grad_weight, int G, const Geo& geo) {
    need_geo(geo); need4d(grad_inputL, "grad_inputL");
    const int dev = check_all({{"grad_outputL", grad_outputL, false}, {"grad_outputU", grad_outputU, false},
                               {"posL", posL, true}, {"posU", posU, true}, {"grad_inputL", grad_inputL, false},
                               {"grad_inputU", grad_inputU, false}, {"grad_weight", grad_weight, false}});
    Launch L(dev);
    raise_on(ndist_conv_bound_inf_dist_backward_input_weight(F(grad_outputL), F(grad_outputU), I(posL), I(posU),
                                                             IMG4(grad_inputL), (int)grad_weight.size(0), G, GEO8(geo),
                                                             FM(grad_inputL), FM(grad_inputU), FM(grad_weight), L.stream),
             "conv_bound_inf_dist_backward_input_weight");
}

// ---- mean shift and bias (no kernel of its own in the reference: core/modules/basic_modules.py:121-132) ------------
// absent tensors are passed as None
using OptTensor = c10::optional<Tensor>;
const float* FO(const OptTensor& t) { return t.has_value() ? t->data_ptr<float>() : nullptr; }
float* FMO(OptTensor& t) { return t.has_value() ? t->data_ptr<float>() : nullptr; }

int check_optional(std::initializer_list<std::pair<const char*, const OptTensor*>> args) {
    int dev = -1;
    for (const auto& a : args) {
        if (!a.second->has_value()) continue;
        const Tensor& t = **a.second;
        TORCH_CHECK(t.is_cuda(), a.first, " must be a CUDA tensor");
        TORCH_CHECK(t.is_contiguous(), a.first, " must be contiguous");
        TORCH_CHECK(t.scalar_type() == torch::kFloat32, a.first, " must have dtype torch.float32");
        if (dev < 0) dev = t.get_device();
        TORCH_CHECK(t.get_device() == dev, a.first, " is on device ", t.get_device(), ", expected ", dev);
    }
    TORCH_CHECK(dev >= 0, "at least one tensor is required");
    return dev;
}

void mean_shift_forward(const OptTensor& x, const OptTensor& lower, const OptTensor& upper, int B, int C, int HW,
                        bool training, double momentum, OptTensor running_mean, const OptTensor& bias1,
                        const OptTensor& bias2, OptTensor mean_out, OptTensor y, OptTensor y_lower, OptTensor y_upper) {
    const int dev = check_optional({{"x", &x}, {"lower", &lower}, {"upper", &upper}, {"running_mean", &running_mean},
                                    {"bias1", &bias1}, {"bias2", &bias2}, {"mean_out", &mean_out}, {"y", &y},
                                    {"y_lower", &y_lower}, {"y_upper", &y_upper}});
    Launch L(dev);
    raise_on(ndist_mean_shift_forward(FO(x), FO(lower), FO(upper), B, C, HW, training ? 1 : 0, (float)momentum,
                                      FMO(running_mean), FO(bias1), FO(bias2), FMO(mean_out), FMO(y), FMO(y_lower),
                                      FMO(y_upper), L.stream), "mean_shift_forward");
}

void mean_shift_backward(const OptTensor& grad_y, const OptTensor& grad_y_lower, const OptTensor& grad_y_upper, int B,
                         int C, int HW, bool training, OptTensor grad_x, OptTensor colsum_out, OptTensor mean_scratch) {
    const int dev = check_optional({{"grad_y", &grad_y}, {"grad_y_lower", &grad_y_lower}, {"grad_y_upper", &grad_y_upper},
                                    {"grad_x", &grad_x}, {"colsum_out", &colsum_out}, {"mean_scratch", &mean_scratch}});
    Launch L(dev);
    raise_on(ndist_mean_shift_backward(FO(grad_y), FO(grad_y_lower), FO(grad_y_upper), B, C, HW, training ? 1 : 0,
                                       FMO(grad_x), FMO(colsum_out), FMO(mean_scratch), L.stream), "mean_shift_backward");
}

// ---- process-wide switches and aids ------------------------------------------------------------------------------
double last_kernel_ms() {
    float ms = 0.f;
    raise_on(ndist_last_kernel_ms(&ms), "last_kernel_ms");
    return ms;
}
std::pair<long, long> scratch_counters() {
    long m = 0, f = 0;
    ndist_scratch_counters(&m, &f);
    return {m, f};
}
void release_scratch() { raise_on(ndist_release_scratch(), "release_scratch"); }

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "L_p-distance operator for MI355X: PyTorch binding over libnorm_dist_hip.so";
    // the reference's twelve (core/cuda/norm_dist.cpp:191-204)
    m.def("norm_dist_forward", &norm_dist_forward);
    m.def("norm_dist_forward_with_max", &norm_dist_forward_with_max);
    m.def("norm_dist_backward_input", &norm_dist_backward_input);
    m.def("norm_dist_backward_input_weight", &norm_dist_backward_input_weight);
    m.def("inf_dist_forward", &inf_dist_forward);
    m.def("inf_dist_forward_nograd", &inf_dist_forward_nograd);
    m.def("inf_dist_backward_input", &inf_dist_backward_input);
    m.def("inf_dist_backward_input_weight", &inf_dist_backward_input_weight);
    m.def("bound_inf_dist_forward", &bound_inf_dist_forward);
    m.def("bound_inf_dist_forward_nograd", &bound_inf_dist_forward_nograd);
    m.def("bound_inf_dist_backward_input", &bound_inf_dist_backward_input);
    m.def("bound_inf_dist_backward_input_weight", &bound_inf_dist_backward_input_weight);
    // additions of this library
    m.def("norm_dist_backward_input_weight_noalloc", &norm_dist_backward_input_weight_noalloc);
    m.def("unfold_forward", &unfold_forward);
    m.def("unfold_backward", &unfold_backward);
    m.def("conv_inf_dist_forward_nograd", &conv_inf_dist_forward_nograd);
    m.def("conv_bound_inf_dist_forward_nograd", &conv_bound_inf_dist_forward_nograd);
    m.def("conv_inf_dist_forward", &conv_inf_dist_forward);
    m.def("conv_norm_dist_forward", &conv_norm_dist_forward);
    m.def("conv_norm_dist_backward_input", &conv_norm_dist_backward_input);
    m.def("conv_norm_dist_backward_input_weight", &conv_norm_dist_backward_input_weight);
    m.def("conv_bound_inf_dist_forward", &conv_bound_inf_dist_forward);
    m.def("conv_inf_dist_backward_input", &conv_inf_dist_backward_input);
    m.def("conv_inf_dist_backward_input_weight", &conv_inf_dist_backward_input_weight);
    m.def("conv_bound_inf_dist_backward_input", &conv_bound_inf_dist_backward_input);
    m.def("conv_bound_inf_dist_backward_input_weight", &conv_bound_inf_dist_backward_input_weight);
    m.def("inf_and_bound_forward_nograd", &inf_and_bound_forward_nograd);
    m.def("inf_and_bound_forward", &inf_and_bound_forward);
    m.def("mean_shift_forward", &mean_shift_forward);
    m.def("mean_shift_backward", &mean_shift_backward);
    m.def("version", []() { return ndist_version(); });
    m.def("set_profiling", [](bool on) { ndist_set_profiling(on ? 1 : 0); });
    m.def("last_kernel_ms", &last_kernel_ms);
    m.def("set_skip_mode", [](int skip, int bounds) { ndist_set_skip_mode(skip, bounds); });
    m.def("set_hot_mode", [](int mode) { ndist_set_hot_mode(mode); });
    m.def("set_scaled_mode", [](int mode) { ndist_set_scaled_mode(mode); });
    m.def("release_scratch", &release_scratch);
    m.def("scratch_counters", &scratch_counters);
    m.def("noalloc_scratch_bytes", []() { return (long)ndist_noalloc_scratch_bytes(); });
}
