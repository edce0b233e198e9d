// mmcv_amd._ext: the PyTorch-ROCm side of the drop-in boundary.  It exports the
// two ops mmcv's Python layer asserts on
// (mmcv/ops/modulated_deform_conv.py:17-19, mmcv/utils/ext_loader.py:12-16) with
// the signature and keyword names of mmcv/ops/csrc/pytorch/pybind.cpp:157-170,
// 641-657, and forwards device tensors to the C ABI of libmdcn_hip.so.
//
// There is no CPU implementation here on purpose: a call with CPU tensors
// raises, the way the reference's device registry does for a device nobody
// registered (mmcv/ops/csrc/common/pytorch_device_registry.hpp:120-126).
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <string>
#include <vector>

#include <atomic>

#include "mdcn.h"

namespace {

using at::Tensor;

// device path of every op of this module (set_path); read once per call
std::atomic<int> g_path{MDCN_PATH_AUTO};
// mdcn_params.no_k_split of every forward of this module (set_k_split)
std::atomic<int> g_no_k_split{0};

std::string device_str(const at::Device &d) {
  std::string s = c10::DeviceTypeName(d.type(), /*lower_case=*/true);
  if (d.has_index()) s += ":" + std::to_string(d.index());
  return s;
}

int mdcn_dtype_of(const Tensor &t) {
  switch (t.scalar_type()) {
    case at::kFloat: return MDCN_F32;
    case at::kHalf: return MDCN_F16;
    case at::kBFloat16: return MDCN_BF16;
    case at::kDouble: return MDCN_F64;
    default:
      TORCH_CHECK(false, "\"modulated_deform_conv_forward\" not implemented for '",
                  c10::toString(t.scalar_type()), "'");
  }
}

struct Prepared {
  mdcn_params p;
  std::vector<Tensor> keep;  // contiguous copies and the workspace
};

// Checks in the order of the reference host op
// (mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:68-90), then the dispatch
// checks (pytorch_device_registry.hpp:115-128).
// false: the batch is empty and there is nothing to do (the reference's loop over
// samples, modulated_deform_conv.cpp:108-130, runs zero times)
bool prepare(Prepared &pr, const Tensor &input, const Tensor &weight,
             const Tensor &bias, const Tensor &offset, const Tensor &mask,
             Tensor &output, int kernel_h, int kernel_w, int stride_h,
             int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w,
             int group, int deformable_group, bool with_bias) {
  TORCH_CHECK(input.dim() == 4 && weight.dim() == 4 && offset.dim() == 4 &&
                  mask.dim() == 4,
              "modulated_deform_conv_forward expects 4-D input, weight, offset and mask");
  const int64_t batch = input.size(0), channels = input.size(1);
  const int64_t height = input.size(2), width = input.size(3);
  const int64_t channels_out = weight.size(0), channels_kernel = weight.size(1);
  TORCH_CHECK(weight.size(2) == kernel_h && weight.size(3) == kernel_w,
              "Input shape and kernel shape won't match: (", kernel_h, " x ",
              kernel_w, " vs ", weight.size(2), " x ", weight.size(3), ").");
  TORCH_CHECK(channels == channels_kernel * group,
              "Input shape and kernel channels won't match: (", channels, " vs ",
              channels_kernel * group, ").");

  const at::Device dev = input.device();
  TORCH_CHECK(dev.is_cuda(),
              "modulated_deformable_im2col_impl: implementation for device ",
              device_str(dev), " not found.");
  const Tensor *all[] = {&input, &weight, &bias, &offset, &mask, &output};
  const char *names[] = {"input", "weight", "bias", "offset", "mask", "output"};
  for (int i = 1; i < 6; ++i)
    TORCH_CHECK(all[i]->device() == dev, "modulated_deform_conv_forward: at param ",
                names[i], ", inconsistent device: ", device_str(all[i]->device()),
                " vs ", device_str(dev));
  const auto st = input.scalar_type();
  for (int i = 1; i < 6; ++i)
    TORCH_CHECK(all[i]->scalar_type() == st,
                "modulated_deform_conv_forward: expected ", names[i],
                " to have dtype ", c10::toString(st), " but got ",
                c10::toString(all[i]->scalar_type()));
  if (batch == 0) return false;

  mdcn_params &p = pr.p;
  p = mdcn_params{};
  p.dtype = mdcn_dtype_of(input);
  p.path = g_path.load();
  p.no_k_split = g_no_k_split.load();
  p.N = (int)batch; p.Cin = (int)channels; p.H = (int)height; p.W = (int)width;
  p.Cout = (int)channels_out; p.kh = kernel_h; p.kw = kernel_w;
  p.sh = stride_h; p.sw = stride_w; p.ph = pad_h; p.pw = pad_w;
  p.dh = dilation_h; p.dw = dilation_w;
  p.groups = group; p.dgroups = deformable_group;

  int32_t Ho = 0, Wo = 0;
  const int rc = mdcn_output_size(&p, &Ho, &Wo);
  TORCH_CHECK(rc == MDCN_OK, "modulated_deform_conv_forward: ", mdcn_status_string(rc));
  const int64_t taps = (int64_t)kernel_h * kernel_w;
  TORCH_CHECK(offset.size(0) == batch && offset.size(1) == deformable_group * 2 * taps &&
                  offset.size(2) == Ho && offset.size(3) == Wo,
              "modulated_deform_conv_forward: offset must be (", batch, ", ",
              deformable_group * 2 * taps, ", ", Ho, ", ", Wo, "), got ", offset.sizes());
  TORCH_CHECK(mask.size(0) == batch && mask.size(1) == deformable_group * taps &&
                  mask.size(2) == Ho && mask.size(3) == Wo,
              "modulated_deform_conv_forward: mask must be (", batch, ", ",
              deformable_group * taps, ", ", Ho, ", ", Wo, "), got ", mask.sizes());
  TORCH_CHECK(output.numel() == batch * channels_out * Ho * Wo && output.is_contiguous(),
              "modulated_deform_conv_forward: output must be a dense (", batch, ", ",
              channels_out, ", ", Ho, ", ", Wo, ") tensor, got ", output.sizes());
  if (with_bias)
    TORCH_CHECK(bias.numel() == channels_out,
                "modulated_deform_conv_forward: bias must have ", channels_out,
                " elements, got ", bias.numel());

  auto dense = [&](const Tensor &t) {
    pr.keep.push_back(t.contiguous());
    return pr.keep.back().data_ptr();
  };
  // a channels-last input is read in place when the fused kernel covers the shape
  p.input = nullptr;
  if (!input.is_contiguous() && input.is_contiguous(at::MemoryFormat::ChannelsLast)) {
    p.input = input.data_ptr();
    p.input_nhwc = 1;
    if (!mdcn_fused_eligible(&p) || p.path == MDCN_PATH_DIRECT) {
      p.input = nullptr;
      p.input_nhwc = 0;
    }
  }
  if (!p.input) p.input = dense(input);
  p.offset = dense(offset);
  p.mask = dense(mask);
  p.weight = dense(weight);
  p.bias = with_bias ? dense(bias) : nullptr;
  p.output = output.data_ptr();

  const size_t ws = mdcn_workspace_bytes(&p);
  if (ws > 0) {
    // torch's caching allocator: stream-ordered with the launches below
    pr.keep.push_back(at::empty({(int64_t)ws}, input.options().dtype(at::kByte)));
    p.workspace = pr.keep.back().data_ptr();
    p.workspace_bytes = ws;
  }
  return true;
}

void modulated_deform_conv_forward(
    Tensor input, Tensor weight, Tensor bias, Tensor ones, Tensor offset,
    Tensor mask, Tensor output, Tensor columns, int kernel_h, int kernel_w,
    const int stride_h, const int stride_w, const int pad_h, const int pad_w,
    const int dilation_h, const int dilation_w, const int group,
    const int deformable_group, const bool with_bias) {
  // `ones` and `columns` are the reference's scratch placeholders
  // (mmcv/ops/modulated_deform_conv.py:149); the fused path has no use for them.
  (void)ones;
  (void)columns;
  c10::DeviceGuard guard(input.device());
  Prepared pr;
  if (!prepare(pr, input, weight, bias, offset, mask, output, kernel_h, kernel_w,
               stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, group,
               deformable_group, with_bias))
    return;
  void *stream = (void *)c10::hip::getCurrentHIPStream().stream();
  const int rc = mdcn_forward(&pr.p, stream);
  TORCH_CHECK(rc == MDCN_OK, "modulated_deform_conv_forward: ", mdcn_status_string(rc));
}

// Same call, timed stage by stage with HIP events on the current stream.
std::vector<double> modulated_deform_conv_forward_timed(
    Tensor input, Tensor weight, Tensor bias, Tensor offset, Tensor mask,
    Tensor output, int kernel_h, int kernel_w, int stride_h, int stride_w,
    int pad_h, int pad_w, int dilation_h, int dilation_w, int group,
    int deformable_group, bool with_bias) {
  c10::DeviceGuard guard(input.device());
  Prepared pr;
  if (!prepare(pr, input, weight, bias, offset, mask, output, kernel_h, kernel_w,
               stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, group,
               deformable_group, with_bias))
    return {0, 0, 0, 0};
  void *stream = (void *)c10::hip::getCurrentHIPStream().stream();
  float ms[4] = {0, 0, 0, 0};
  const int rc = mdcn_forward_timed(&pr.p, stream, ms);
  TORCH_CHECK(rc == MDCN_OK, "modulated_deform_conv_forward: ", mdcn_status_string(rc));
  return {ms[0], ms[1], ms[2], ms[3]};
}

// ModulatedDeformConv2dPack.forward in one call
// (mmcv/ops/modulated_deform_conv.py:327-335): conv_offset, the channel split,
// the sigmoid and the deformable convolution.  `offset_weight` with zero
// elements means that `raw` already holds the conv_offset output (computed by
// the caller); otherwise conv_offset runs here and `raw`, when it has elements,
// receives its output.  Returns per-stage milliseconds when `timed`.
std::vector<double> modulated_deform_conv_pack_forward(
    Tensor input, Tensor offset_weight, Tensor offset_bias, Tensor raw,
    Tensor weight, Tensor bias, Tensor output, int kernel_h, int kernel_w,
    int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h,
    int dilation_w, int group, int deformable_group, bool with_bias, bool timed,
    bool unmodulated) {
  const char *op = "modulated_deform_conv_pack_forward";
  TORCH_CHECK(input.dim() == 4 && weight.dim() == 4, op, " expects 4-D input and weight");
  const at::Device dev = input.device();
  TORCH_CHECK(dev.is_cuda(), op, ": implementation for device ", device_str(dev), " not found.");
  c10::DeviceGuard guard(dev);
  const int64_t batch = input.size(0), channels = input.size(1);
  const int64_t channels_out = weight.size(0);
  TORCH_CHECK(weight.size(2) == kernel_h && weight.size(3) == kernel_w,
              "Input shape and kernel shape won't match: (", kernel_h, " x ", kernel_w,
              " vs ", weight.size(2), " x ", weight.size(3), ").");
  TORCH_CHECK(channels == weight.size(1) * group,
              "Input shape and kernel channels won't match: (", channels, " vs ",
              weight.size(1) * group, ").");
  const bool own_conv = offset_weight.numel() > 0;
  const auto st = input.scalar_type();
  const Tensor *all[] = {&weight, &bias, &output, &offset_weight, &offset_bias, &raw};
  const char *names[] = {"weight", "bias", "output", "offset_weight", "offset_bias", "raw"};
  for (int i = 0; i < 6; ++i) {
    if (all[i]->numel() == 0) continue;
    TORCH_CHECK(all[i]->device() == dev, op, ": at param ", names[i], ", inconsistent device: ",
                device_str(all[i]->device()), " vs ", device_str(dev));
    TORCH_CHECK(all[i]->scalar_type() == st, op, ": expected ", names[i], " to have dtype ",
                c10::toString(st), " but got ", c10::toString(all[i]->scalar_type()));
  }
  if (batch == 0) return {0, 0, 0, 0, 0};  // nothing to compute, nothing to write

  mdcn_pack_params pp{};
  mdcn_params &p = pp.conv;
  p.dtype = mdcn_dtype_of(input);
  p.path = g_path.load();
  p.no_k_split = g_no_k_split.load();
  p.N = (int)batch; p.Cin = (int)channels; p.H = (int)input.size(2); p.W = (int)input.size(3);
  p.Cout = (int)channels_out; p.kh = kernel_h; p.kw = kernel_w;
  p.sh = stride_h; p.sw = stride_w; p.ph = pad_h; p.pw = pad_w;
  p.dh = dilation_h; p.dw = dilation_w;
  p.groups = group; p.dgroups = deformable_group;
  int32_t Ho = 0, Wo = 0;
  int rc = mdcn_output_size(&p, &Ho, &Wo);
  TORCH_CHECK(rc == MDCN_OK, op, ": ", mdcn_status_string(rc));
  const int64_t co = (int64_t)(unmodulated ? 2 : 3) * deformable_group * kernel_h * kernel_w;
  pp.unmodulated = unmodulated ? 1 : 0;
  TORCH_CHECK(output.numel() == batch * channels_out * Ho * Wo && output.is_contiguous(), op,
              ": output must be a dense (", batch, ", ", channels_out, ", ", Ho, ", ", Wo,
              ") tensor, got ", output.sizes());
  if (own_conv) {
    TORCH_CHECK(offset_weight.dim() == 4 && offset_weight.size(0) == co &&
                    offset_weight.size(1) == channels && offset_weight.size(2) == kernel_h &&
                    offset_weight.size(3) == kernel_w,
                op, ": offset_weight must be (", co, ", ", channels, ", ", kernel_h, ", ",
                kernel_w, "), got ", offset_weight.sizes());
    TORCH_CHECK(offset_bias.numel() == 0 || offset_bias.numel() == co, op,
                ": offset_bias must have ", co, " elements, got ", offset_bias.numel());
  } else {
    TORCH_CHECK(raw.numel() > 0, op, ": needs offset_weight or raw");
  }
  if (raw.numel() > 0)
    TORCH_CHECK(raw.dim() == 4 && raw.size(0) == batch && raw.size(1) == co && raw.size(2) == Ho &&
                    raw.size(3) == Wo && (own_conv ? raw.is_contiguous() : true),
                op, ": raw must be a dense (", batch, ", ", co, ", ", Ho, ", ", Wo,
                ") tensor, got ", raw.sizes());
  if (with_bias)
    TORCH_CHECK(bias.numel() == channels_out, op, ": bias must have ", channels_out,
                " elements, got ", bias.numel());

  std::vector<Tensor> keep;
  auto dense = [&](const Tensor &t) {
    keep.push_back(t.contiguous());
    return keep.back().data_ptr();
  };
  p.input = dense(input);
  p.weight = dense(weight);
  p.bias = with_bias ? dense(bias) : nullptr;
  p.output = output.data_ptr();
  if (own_conv) {
    pp.offset_weight = dense(offset_weight);
    pp.offset_bias = offset_bias.numel() ? dense(offset_bias) : nullptr;
    pp.raw = raw.numel() ? raw.data_ptr() : nullptr;
  } else {
    pp.raw = dense(raw);
  }
  const size_t ws = mdcn_pack_workspace_bytes(&pp);
  if (ws > 0) {
    keep.push_back(at::empty({(int64_t)ws}, input.options().dtype(at::kByte)));
    p.workspace = keep.back().data_ptr();
    p.workspace_bytes = ws;
  }
  void *stream = (void *)c10::hip::getCurrentHIPStream().stream();
  float ms[5] = {0, 0, 0, 0, 0};
  rc = timed ? mdcn_pack_forward_timed(&pp, stream, ms) : mdcn_pack_forward(&pp, stream);
  TORCH_CHECK(rc == MDCN_OK, op, ": ", mdcn_status_string(rc));
  return {ms[0], ms[1], ms[2], ms[3], ms[4]};
}

// Deformable convolution without modulation
// (mmcv/ops/csrc/pytorch/deform_conv.cpp:140-260; pybind.cpp:38-62,525-547 for the
// argument names).  `columns`, `ones` and `im2col_step` size the reference's
// scratch buffers and are not needed here; the step must still divide the batch,
// as its caller asserts (mmcv/ops/deform_conv.py:115-117).
void deform_conv_forward(Tensor input, Tensor weight, Tensor offset, Tensor output,
                         Tensor columns, Tensor ones, int kW, int kH, int dW, int dH,
                         int padW, int padH, int dilationW, int dilationH, int group,
                         int deformable_group, int im2col_step) {
  (void)columns;
  (void)ones;
  const char *op = "deform_conv_forward";
  TORCH_CHECK(weight.dim() == 4, "4D weight tensor (nOutputPlane,nInputPlane,kH,kW) expected, but got: ",
              weight.dim());
  TORCH_CHECK(kW > 0 && kH > 0, "kernel size should be greater than zero, but got kH: ", kH, " kW: ", kW);
  TORCH_CHECK(weight.size(2) == kH && weight.size(3) == kW,
              "kernel size should be consistent with weight, but got kH: ", kH, " kW: ", kW,
              " weight.size(2): ", weight.size(2), ", weight.size(3): ", weight.size(3));
  TORCH_CHECK(dW > 0 && dH > 0, "stride should be greater than zero, but got dH: ", dH, " dW: ", dW);
  TORCH_CHECK(dilationW > 0 && dilationH > 0, "dilation should be greater than 0, but got dilationH: ",
              dilationH, " dilationW: ", dilationW);
  TORCH_CHECK(input.dim() == 3 || input.dim() == 4, "3D or 4D input tensor expected but got: ", input.dim());
  if (input.dim() == 3) {  // the reference forces a batch of one (:171-176)
    input = input.unsqueeze(0);
    offset = offset.unsqueeze(0);
  }
  TORCH_CHECK(offset.dim() == 4, op, " expects a 4-D offset");
  const int64_t batch = input.size(0), planes = weight.size(1) * group;
  TORCH_CHECK(planes % deformable_group == 0, "input channels must divide deformable group size");
  TORCH_CHECK(input.size(1) == planes, "invalid number of input planes, expected: ", planes,
              ", but got: ", input.size(1));
  TORCH_CHECK(input.size(2) >= kH && input.size(3) >= kW, "input image is smaller than kernel");
  TORCH_CHECK(im2col_step > 0 && batch % im2col_step == 0, op,
              ": batch size must be divisible by im2col_step");
  const at::Device dev = input.device();
  TORCH_CHECK(dev.is_cuda(), "deformable_im2col_impl: implementation for device ", device_str(dev),
              " not found.");
  c10::DeviceGuard guard(dev);
  const auto st = input.scalar_type();
  const Tensor *all[] = {&weight, &offset, &output};
  const char *names[] = {"weight", "offset", "output"};
  for (int i = 0; i < 3; ++i) {
    TORCH_CHECK(all[i]->device() == dev, op, ": at param ", names[i], ", inconsistent device: ",
                device_str(all[i]->device()), " vs ", device_str(dev));
    TORCH_CHECK(all[i]->scalar_type() == st, op, ": expected ", names[i], " to have dtype ",
                c10::toString(st), " but got ", c10::toString(all[i]->scalar_type()));
  }
  mdcn_params p{};
  p.dtype = mdcn_dtype_of(input);
  p.path = g_path.load();
  p.no_k_split = g_no_k_split.load();
  p.N = (int)batch; p.Cin = (int)planes; p.H = (int)input.size(2); p.W = (int)input.size(3);
  p.Cout = (int)weight.size(0); p.kh = kH; p.kw = kW;
  p.sh = dH; p.sw = dW; p.ph = padH; p.pw = padW; p.dh = dilationH; p.dw = dilationW;
  p.groups = group; p.dgroups = deformable_group;
  int32_t Ho = 0, Wo = 0;
  int rc = mdcn_output_size(&p, &Ho, &Wo);
  TORCH_CHECK(rc == MDCN_OK, "Given input size: (", planes, " x ", input.size(2), " x ", input.size(3),
              "). Output size is too small");
  TORCH_CHECK(offset.size(0) == batch, "invalid batch size of offset");
  TORCH_CHECK(offset.size(2) == Ho && offset.size(3) == Wo,
              "invalid spatial size of offset, expected height: ", Ho, " width: ", Wo,
              ", but got height: ", offset.size(2), " width: ", offset.size(3));
  TORCH_CHECK(offset.size(1) == (int64_t)deformable_group * 2 * kH * kW,
              "invalid number of channels of offset");
  TORCH_CHECK(output.numel() == batch * weight.size(0) * Ho * Wo && output.is_contiguous(), op,
              ": output must be a dense (", batch, ", ", weight.size(0), ", ", Ho, ", ", Wo,
              ") tensor, got ", output.sizes());
  std::vector<Tensor> keep = {input.contiguous(), offset.contiguous(), weight.contiguous()};
  p.input = keep[0].data_ptr();
  p.offset = keep[1].data_ptr();
  p.mask = nullptr;
  p.weight = keep[2].data_ptr();
  p.bias = nullptr;
  p.output = output.data_ptr();
  const size_t ws = mdcn_workspace_bytes(&p);
  if (ws > 0) {
    keep.push_back(at::empty({(int64_t)ws}, input.options().dtype(at::kByte)));
    p.workspace = keep.back().data_ptr();
    p.workspace_bytes = ws;
  }
  rc = mdcn_forward(&p, (void *)c10::hip::getCurrentHIPStream().stream());
  TORCH_CHECK(rc == MDCN_OK, op, ": ", mdcn_status_string(rc));
}

// Shared by the three backward ops: checks, contiguity, workspace and the call.
// Tensors with zero elements stand for "not wanted".
void run_backward(const char *op, const Tensor &input, const Tensor &weight, const Tensor &offset,
                  const Tensor &mask, const Tensor &grad_output, Tensor grad_input,
                  Tensor grad_offset, Tensor grad_mask, Tensor grad_weight, Tensor grad_bias,
                  int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w,
                  int dilation_h, int dilation_w, int group, int deformable_group) {
  TORCH_CHECK(input.dim() == 4 && weight.dim() == 4 && offset.dim() == 4 && grad_output.dim() == 4, op,
              " expects 4-D input, weight, offset and grad_output");
  const at::Device dev = input.device();
  TORCH_CHECK(dev.is_cuda(), op, ": implementation for device ", device_str(dev), " not found.");
  c10::DeviceGuard guard(dev);
  TORCH_CHECK(weight.size(2) == kernel_h && weight.size(3) == kernel_w,
              "Input shape and kernel shape won't match: (", kernel_h, " x ", kernel_w, " vs ",
              weight.size(2), " x ", weight.size(3), ").");
  TORCH_CHECK(input.size(1) == weight.size(1) * group, "Input shape and kernel channels won't match: (",
              input.size(1), " vs ", weight.size(1) * group, ").");
  const auto st = input.scalar_type();
  const Tensor *all[] = {&weight, &offset, &mask, &grad_output, &grad_input, &grad_offset,
                         &grad_mask, &grad_weight, &grad_bias};
  const char *names[] = {"weight", "offset", "mask", "grad_output", "grad_input", "grad_offset",
                         "grad_mask", "grad_weight", "grad_bias"};
  for (int i = 0; i < 9; ++i) {
    if (all[i]->numel() == 0) continue;
    TORCH_CHECK(all[i]->device() == dev, op, ": at param ", names[i], ", inconsistent device: ",
                device_str(all[i]->device()), " vs ", device_str(dev));
    TORCH_CHECK(all[i]->scalar_type() == st, op, ": expected ", names[i], " to have dtype ",
                c10::toString(st), " but got ", c10::toString(all[i]->scalar_type()));
    if (i >= 4) TORCH_CHECK(all[i]->is_contiguous(), op, ": ", names[i], " must be contiguous");
  }
  if (input.size(0) == 0) {  // no sample contributes: the parameter gradients are zero, the others empty
    if (grad_weight.numel()) grad_weight.zero_();
    if (grad_bias.numel()) grad_bias.zero_();
    return;
  }
  mdcn_bwd_params bp{};
  mdcn_params &p = bp.conv;
  p.dtype = mdcn_dtype_of(input);
  p.N = (int)input.size(0); p.Cin = (int)input.size(1); p.H = (int)input.size(2); p.W = (int)input.size(3);
  p.Cout = (int)weight.size(0); p.kh = kernel_h; p.kw = kernel_w;
  p.sh = stride_h; p.sw = stride_w; p.ph = pad_h; p.pw = pad_w; p.dh = dilation_h; p.dw = dilation_w;
  p.groups = group; p.dgroups = deformable_group;
  p.path = g_path.load();
  p.no_k_split = g_no_k_split.load();
  int32_t Ho = 0, Wo = 0;
  int rc = mdcn_output_size(&p, &Ho, &Wo);
  TORCH_CHECK(rc == MDCN_OK, op, ": ", mdcn_status_string(rc));
  const int64_t taps = (int64_t)kernel_h * kernel_w;
  TORCH_CHECK(grad_output.size(0) == p.N && grad_output.size(1) == p.Cout && grad_output.size(2) == Ho &&
                  grad_output.size(3) == Wo,
              op, ": grad_output must be (", p.N, ", ", p.Cout, ", ", Ho, ", ", Wo, "), got ",
              grad_output.sizes());
  TORCH_CHECK(offset.size(0) == p.N && offset.size(1) == deformable_group * 2 * taps &&
                  offset.size(2) == Ho && offset.size(3) == Wo,
              op, ": offset must be (", p.N, ", ", deformable_group * 2 * taps, ", ", Ho, ", ", Wo,
              "), got ", offset.sizes());
  const bool modulated = mask.numel() > 0;
  if (modulated)
    TORCH_CHECK(mask.size(0) == p.N && mask.size(1) == deformable_group * taps && mask.size(2) == Ho &&
                    mask.size(3) == Wo,
                op, ": mask must be (", p.N, ", ", deformable_group * taps, ", ", Ho, ", ", Wo, "), got ",
                mask.sizes());
  auto same = [&](const Tensor &grad, const Tensor &like, const char *name) {
    TORCH_CHECK(grad.numel() == 0 || grad.numel() == like.numel(), op, ": ", name, " has ", grad.numel(),
                " elements, expected ", like.numel());
  };
  same(grad_input, input, "grad_input");
  same(grad_offset, offset, "grad_offset");
  same(grad_mask, mask, "grad_mask");
  same(grad_weight, weight, "grad_weight");
  TORCH_CHECK(grad_bias.numel() == 0 || grad_bias.numel() == p.Cout, op, ": grad_bias must have ", p.Cout,
              " elements");
  std::vector<Tensor> keep = {input.contiguous(), offset.contiguous(), weight.contiguous(),
                              grad_output.contiguous()};
  p.input = keep[0].data_ptr();
  p.offset = keep[1].data_ptr();
  p.weight = keep[2].data_ptr();
  bp.grad_output = keep[3].data_ptr();
  if (modulated) {
    keep.push_back(mask.contiguous());
    p.mask = keep.back().data_ptr();
  }
  auto ptr = [](Tensor &t) { return t.numel() ? t.data_ptr() : nullptr; };
  bp.grad_input = ptr(grad_input);
  bp.grad_offset = ptr(grad_offset);
  bp.grad_mask = ptr(grad_mask);
  bp.grad_weight = ptr(grad_weight);
  bp.grad_bias = ptr(grad_bias);
  const size_t ws = mdcn_backward_workspace_bytes(&bp);
  if (ws > 0) {
    keep.push_back(at::empty({(int64_t)ws}, input.options().dtype(at::kByte)));
    p.workspace = keep.back().data_ptr();
    p.workspace_bytes = ws;
  }
  rc = mdcn_backward(&bp, (void *)c10::hip::getCurrentHIPStream().stream());
  TORCH_CHECK(rc == MDCN_OK, op, ": ", mdcn_status_string(rc));
}

// mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:140-251.  The reference adds
// into the gradient tensors its caller hands over freshly zeroed
// (mmcv/ops/modulated_deform_conv.py:177-181); here they are overwritten.
void modulated_deform_conv_backward(
    Tensor input, Tensor weight, Tensor bias, Tensor ones, Tensor offset,
    Tensor mask, Tensor columns, Tensor grad_input, Tensor grad_weight,
    Tensor grad_bias, Tensor grad_offset, Tensor grad_mask, Tensor grad_output,
    int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h,
    int pad_w, int dilation_h, int dilation_w, int group, int deformable_group,
    const bool with_bias) {
  (void)bias;
  (void)ones;
  (void)columns;
  run_backward("modulated_deform_conv_backward", input, weight, offset, mask, grad_output, grad_input,
               grad_offset, grad_mask, grad_weight, with_bias ? grad_bias : Tensor(at::empty({0}, input.options())),
               kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, group,
               deformable_group);
}

// mmcv/ops/csrc/pytorch/deform_conv.cpp:262-384: gradients of the unmodulated
// convolution with respect to input and offset.
void deform_conv_backward_input(Tensor input, Tensor offset, Tensor gradOutput, Tensor gradInput,
                                Tensor gradOffset, Tensor weight, Tensor columns, int kW, int kH,
                                int dW, int dH, int padW, int padH, int dilationW, int dilationH,
                                int group, int deformable_group, int im2col_step) {
  (void)columns;
  TORCH_CHECK(im2col_step > 0 && input.size(0) % im2col_step == 0,
              "deform_conv_backward_input: batch size must be divisible by im2col_step");
  const Tensor none = at::empty({0}, input.options());
  run_backward("deform_conv_backward_input", input, weight, offset, none, gradOutput, gradInput,
               gradOffset, none, none, none, kH, kW, dH, dW, padH, padW, dilationH, dilationW, group,
               deformable_group);
}

// mmcv/ops/csrc/pytorch/deform_conv.cpp:386-525: gradWeight += scale * (gradient
// with respect to the weight).
void deform_conv_backward_parameters(Tensor input, Tensor offset, Tensor gradOutput,
                                     Tensor gradWeight, Tensor columns, Tensor ones, int kW, int kH,
                                     int dW, int dH, int padW, int padH, int dilationW,
                                     int dilationH, int group, int deformable_group, float scale,
                                     int im2col_step) {
  (void)columns;
  (void)ones;
  TORCH_CHECK(im2col_step > 0 && input.size(0) % im2col_step == 0,
              "deform_conv_backward_parameters: batch size must be divisible by im2col_step");
  const Tensor none = at::empty({0}, input.options());
  Tensor gw = at::empty_like(gradWeight, gradWeight.options(), at::MemoryFormat::Contiguous);
  run_backward("deform_conv_backward_parameters", input, gradWeight, offset, none, gradOutput, none,
               none, none, gw, none, kH, kW, dH, dW, padH, padW, dilationH, dilationW, group,
               deformable_group);
  gradWeight.add_(gw, scale);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("modulated_deform_conv_forward", &modulated_deform_conv_forward,
        "modulated deform conv forward", py::arg("input"), py::arg("weight"),
        py::arg("bias"), py::arg("ones"), py::arg("offset"), py::arg("mask"),
        py::arg("output"), py::arg("columns"), py::arg("kernel_h"),
        py::arg("kernel_w"), py::arg("stride_h"), py::arg("stride_w"),
        py::arg("pad_h"), py::arg("pad_w"), py::arg("dilation_h"),
        py::arg("dilation_w"), py::arg("group"), py::arg("deformable_group"),
        py::arg("with_bias"));
  m.def("modulated_deform_conv_pack_forward", &modulated_deform_conv_pack_forward,
        "conv_offset + chunk/cat/sigmoid + modulated deform conv forward", py::arg("input"),
        py::arg("offset_weight"), py::arg("offset_bias"), py::arg("raw"), py::arg("weight"),
        py::arg("bias"), py::arg("output"), py::arg("kernel_h"), py::arg("kernel_w"),
        py::arg("stride_h"), py::arg("stride_w"), py::arg("pad_h"), py::arg("pad_w"),
        py::arg("dilation_h"), py::arg("dilation_w"), py::arg("group"),
        py::arg("deformable_group"), py::arg("with_bias"), py::arg("timed") = false,
        py::arg("unmodulated") = false);
  m.def("deform_conv_forward", &deform_conv_forward, "deform_conv_forward", py::arg("input"),
        py::arg("weight"), py::arg("offset"), py::arg("output"), py::arg("columns"), py::arg("ones"),
        py::arg("kW"), py::arg("kH"), py::arg("dW"), py::arg("dH"), py::arg("padW"), py::arg("padH"),
        py::arg("dilationW"), py::arg("dilationH"), py::arg("group"), py::arg("deformable_group"),
        py::arg("im2col_step"));
  m.def("deform_conv_backward_input", &deform_conv_backward_input, "deform_conv_backward_input",
        py::arg("input"), py::arg("offset"), py::arg("gradOutput"), py::arg("gradInput"),
        py::arg("gradOffset"), py::arg("weight"), py::arg("columns"), py::arg("kW"), py::arg("kH"),
        py::arg("dW"), py::arg("dH"), py::arg("padW"), py::arg("padH"), py::arg("dilationW"),
        py::arg("dilationH"), py::arg("group"), py::arg("deformable_group"), py::arg("im2col_step"));
  m.def("deform_conv_backward_parameters", &deform_conv_backward_parameters,
        "deform_conv_backward_parameters", py::arg("input"), py::arg("offset"), py::arg("gradOutput"),
        py::arg("gradWeight"), py::arg("columns"), py::arg("ones"), py::arg("kW"), py::arg("kH"),
        py::arg("dW"), py::arg("dH"), py::arg("padW"), py::arg("padH"), py::arg("dilationW"),
        py::arg("dilationH"), py::arg("group"), py::arg("deformable_group"), py::arg("scale"),
        py::arg("im2col_step"));
  m.def("modulated_deform_conv_backward", &modulated_deform_conv_backward,
        "modulated deform conv backward", py::arg("input"), py::arg("weight"),
        py::arg("bias"), py::arg("ones"), py::arg("offset"), py::arg("mask"),
        py::arg("columns"), py::arg("grad_input"), py::arg("grad_weight"),
        py::arg("grad_bias"), py::arg("grad_offset"), py::arg("grad_mask"),
        py::arg("grad_output"), py::arg("kernel_h"), py::arg("kernel_w"),
        py::arg("stride_h"), py::arg("stride_w"), py::arg("pad_h"),
        py::arg("pad_w"), py::arg("dilation_h"), py::arg("dilation_w"),
        py::arg("group"), py::arg("deformable_group"), py::arg("with_bias"));
  m.def("modulated_deform_conv_forward_timed", &modulated_deform_conv_forward_timed,
        "forward with per-stage HIP-event timing; returns [relayout, pack, main, total] ms",
        py::arg("input"), py::arg("weight"), py::arg("bias"), py::arg("offset"),
        py::arg("mask"), py::arg("output"), py::arg("kernel_h"), py::arg("kernel_w"),
        py::arg("stride_h"), py::arg("stride_w"), py::arg("pad_h"), py::arg("pad_w"),
        py::arg("dilation_h"), py::arg("dilation_w"), py::arg("group"),
        py::arg("deformable_group"), py::arg("with_bias"));
  m.def("set_path", [](int path) {
          TORCH_CHECK(path >= MDCN_PATH_AUTO && path <= MDCN_PATH_FUSED_NARROW,
                      "path must be 0 (auto), 1 (fused), 2 (direct), 3 (fused, specialised-wave kernel only), "
                      "4 (fused, 256-pixel kernel on every whole tile) or 5 (fused, without the 256-pixel kernel)");
          g_path.store(path);
        }, "choose the device path of forward and backward: 0 auto, 1 fused / matrix-core kernels, 2 direct kernels, "
           "3 fused with the specialised-wave forward kernel, 4 fused with the 256-pixel forward kernel on every "
           "whole tile, 5 fused without that kernel", py::arg("path"));
  m.def("get_path", []() { return g_path.load(); });
  m.def("set_k_split", [](bool on) { g_no_k_split.store(on ? 0 : 1); },
        "true (default): idle workgroups of the fused forward kernel's last round take parts of the K range of its "
        "tiles; false: every tile is one fp32 sum formed by one workgroup", py::arg("on"));
  m.def("get_k_split", []() { return g_no_k_split.load() == 0; });
  m.def("abi_version", []() { return mdcn_abi_version(); });
}
