// TEST INFRASTRUCTURE ONLY.  Python binding for the REFERENCE's own
// modulated_deform_conv_forward, compiled from the reference's source files where
// they lie (see the Makefile next to this file).  It lets the tests and the
// benchmark's CPU-baseline leg call mmcv's real CPU path.  The prototype below
// is the one declared in mmcv/ops/csrc/pytorch/pybind.cpp:157-162 and defined in
// mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:395-412; argument names follow
// mmcv/ops/csrc/pytorch/pybind.cpp:641-648.
#include <torch/extension.h>

void modulated_deform_conv_forward(
    at::Tensor input, at::Tensor weight, at::Tensor bias, at::Tensor ones,
    at::Tensor offset, at::Tensor mask, at::Tensor output, at::Tensor columns,
    int kernel_h, int kernel_w, const int stride_h, const int stride_w,
    const int pad_h, const int pad_w, const int dilation_h,
    const int dilation_w, const int group, const int deformable_group,
    const bool with_bias);

// mmcv/ops/csrc/pytorch/pybind.cpp:164-170 (declaration), :649-657 (argument names);
// defined in mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:414-434.
void modulated_deform_conv_backward(
    at::Tensor input, at::Tensor weight, at::Tensor bias, at::Tensor ones,
    at::Tensor offset, at::Tensor mask, at::Tensor columns, at::Tensor grad_input,
    at::Tensor grad_weight, at::Tensor grad_bias, at::Tensor grad_offset,
    at::Tensor grad_mask, at::Tensor grad_output, int kernel_h, int kernel_w,
    int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h,
    int dilation_w, int group, int deformable_group, const bool with_bias);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("modulated_deform_conv_backward", &modulated_deform_conv_backward,
        py::arg("input"), py::arg("weight"), py::arg("bias"), py::arg("ones"),
        py::arg("offset"), py::arg("mask"), py::arg("columns"),
        py::arg("grad_input"), py::arg("grad_weight"), py::arg("grad_bias"),
        py::arg("grad_offset"), py::arg("grad_mask"), py::arg("grad_output"),
        py::arg("kernel_h"), py::arg("kernel_w"), py::arg("stride_h"),
        py::arg("stride_w"), py::arg("pad_h"), py::arg("pad_w"),
        py::arg("dilation_h"), py::arg("dilation_w"), py::arg("group"),
        py::arg("deformable_group"), py::arg("with_bias"));
  m.def("modulated_deform_conv_forward", &modulated_deform_conv_forward,
        py::arg("input"), py::arg("weight"), py::arg("bias"), py::arg("ones"),
        py::arg("offset"), py::arg("mask"), py::arg("output"),
        py::arg("columns"), py::arg("kernel_h"), py::arg("kernel_w"),
        py::arg("stride_h"), py::arg("stride_w"), py::arg("pad_h"),
        py::arg("pad_w"), py::arg("dilation_h"), py::arg("dilation_w"),
        py::arg("group"), py::arg("deformable_group"), py::arg("with_bias"));
}
