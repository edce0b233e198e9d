/*
 * mdcn.h -- C ABI of libmdcn_hip.so: modulated deformable convolution (DCNv2)
 * forward for AMD MI355X (gfx950), written directly in HIP.
 *
 * Plain C types only: device pointers and sizes, no torch types.  None of the
 * calls below allocates device memory, synchronises the stream or throws; all
 * device work is enqueued on the HIP stream the caller passes.
 *
 * What this replaces in the reference (mmcv v2.2.0):
 *   mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:62-138   host op: output
 *       zeroing, the columns scratch, the per-sample im2col launch, the per-group
 *       addmm_ and the bias add,
 *   mmcv/ops/csrc/pytorch/cuda/modulated_deform_conv_cuda.cu:5-32 and
 *   mmcv/ops/csrc/common/cuda/modulated_deform_conv_cuda_kernel.cuh:80-108,186-245
 *       the im2col device kernel and its sampler,
 * i.e. everything below `modulated_deform_conv_forward`
 * (mmcv/ops/csrc/pytorch/pybind.cpp:157-162) once `input.is_cuda()`.
 */
#ifndef MDCN_H_
#define MDCN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MDCN_ABI_VERSION 5

/* Element type of every tensor of a call (the Python wrapper unifies them to
 * offset's dtype, mmcv/ops/modulated_deform_conv.py:136-139). */
enum mdcn_dtype {
  MDCN_F32 = 0,
  MDCN_F16 = 1,
  MDCN_BF16 = 2,
  MDCN_F64 = 3 /* double: the reference dispatches its kernels over it as well
                  (mmcv/ops/csrc/pytorch/cuda/modulated_deform_conv_cuda.cu:16); served by plain
                  one-thread-per-output kernels that compute in double, forward and backward, never by
                  the fused path, and not by the pack-level call (MDCN_ERR_DTYPE there) */
};

/* Which device path runs. */
enum mdcn_path {
  MDCN_PATH_AUTO = 0,   /* fused MFMA kernel when the shape allows, else direct */
  MDCN_PATH_FUSED = 1,  /* fused implicit-GEMM MFMA kernel; error if not eligible */
  MDCN_PATH_DIRECT = 2, /* one thread per output element; any shape */
  MDCN_PATH_FUSED_SPLIT = 3, /* forward only: as MDCN_PATH_FUSED, but always the fused kernel with specialised
                               producer / consumer wavefronts (what fp32 tensors, several deformable groups and
                               tiles narrower than 256 channels run anyway), never the eight-wave streaming
                               kernel that 16-bit 256-channel tiles get by default; for comparisons and tests */
  MDCN_PATH_FUSED_WIDE = 4, /* forward only: as MDCN_PATH_FUSED, and every whole tile of 256 pixels goes to the
                               kernel with 256-pixel tiles where the shape has one (16-bit tensors, one
                               deformable group, 3 to 9 taps, 128 or a multiple of 256 output channels per
                               group (2048 at most in all), an even number of K steps, output planes of a
                               multiple of 8 and at least 64 pixels; input dense or channels-last), however
                               unevenly that fills the chip; MDCN_PATH_FUSED and MDCN_PATH_AUTO give that
                               kernel all tiles or whole rounds of tiles, whichever its measured tile cost
                               says is shorter, and the rest of the pixels to the 128-pixel kernel.  Error if
                               the shape has no such kernel. */
  MDCN_PATH_FUSED_NARROW = 5 /* forward only: as MDCN_PATH_FUSED, never the 256-pixel kernel */
};

enum mdcn_status {
  MDCN_OK = 0,
  MDCN_ERR_NULL = -1,       /* a required pointer is NULL */
  MDCN_ERR_SHAPE = -2,      /* non-positive size, or Cin/Cout not divisible by groups / deform groups */
  MDCN_ERR_DTYPE = -3,      /* dtype is not one of mdcn_dtype */
  MDCN_ERR_WORKSPACE = -4,  /* workspace missing, misaligned or smaller than mdcn_workspace_bytes() */
  MDCN_ERR_PATH = -5,       /* MDCN_PATH_FUSED asked for a shape it does not cover */
  MDCN_ERR_TOO_LARGE = -6,  /* one padded image exceeds the 32-bit byte offsets used on the device */
  MDCN_ERR_LAUNCH = -7,     /* HIP reported a launch error */
  MDCN_ERR_SCRATCH_LIMIT = -8 /* mdcn_forward_noalloc(): the call needs more than MDCN_NOALLOC_SCRATCH_BYTES */
};

/*
 * One forward call.  All tensors are dense, of element type `dtype`, on the
 * device that is current when the call is made:
 *   input  (N, Cin, H, W)                      NCHW
 *   offset (N, dgroups*2*kh*kw, Ho, Wo)        channel 2t = dy, 2t+1 = dx of tap t = i*kw + j
 *   mask   (N, dgroups*kh*kw, Ho, Wo)           or NULL: unmodulated (DCNv1), see below
 *   weight (Cout, Cin/groups, kh, kw)
 *   bias   (Cout) or NULL                      NULL <=> with_bias == false
 *   output (N, Cout, Ho, Wo)                   written in full, need not be initialised
 * with Ho = (H + 2*ph - (dh*(kh-1)+1))/sh + 1 and Wo likewise
 * (mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:87-90).  Sampling positions and
 * bilinear weights are always computed in fp32; products are accumulated in
 * fp32 and rounded once to `dtype` after the bias add.
 *
 * mask == NULL (with bias == NULL) is the deformable convolution without
 * modulation, `deform_conv_forward` of the reference
 * (mmcv/ops/csrc/pytorch/deform_conv.cpp:140-260, sampler
 * cpu/deform_conv.cpp:5-38): the same sampling rule with factor 1.  The
 * reference's im2col_step only sizes its scratch buffers and has no counterpart.
 */
typedef struct mdcn_params {
  const void *input;
  const void *offset;
  const void *mask;
  const void *weight;
  const void *bias;
  void *output;
  void *workspace;        /* device scratch, 256-byte aligned; may be NULL when mdcn_workspace_bytes() == 0 */
  size_t workspace_bytes;
  int32_t dtype;          /* enum mdcn_dtype */
  int32_t path;           /* enum mdcn_path */
  int32_t N, Cin, H, W;
  int32_t Cout, kh, kw;
  int32_t sh, sw, ph, pw, dh, dw;
  int32_t groups, dgroups;
  int32_t input_nhwc;     /* 0: input is dense (N, Cin, H, W).  1: input is dense channels-last, (N, H, W, Cin)
                             in memory (torch.channels_last); the fused kernel then reads it in place, without
                             the re-laid-out copy.  Fused path of mdcn_forward() only (H, W >= 2); every
                             other tensor keeps its layout. */
  int32_t no_k_split;     /* 0: workgroups that would idle in the last round of the fused kernel's schedule
                             take over parts of the K range of that round's tiles (partial sums meet in
                             the workspace, added in a fixed order: results are the same on every run).
                             1: every tile is summed by one workgroup, as a single fp32 sum over K; an
                             image's output then does not depend on where in the batch it sits.  The two
                             settings differ by fp32 rounding of the sums only. */
} mdcn_params;

/* ABI version of the loaded library (== MDCN_ABI_VERSION it was built with). */
int mdcn_abi_version(void);

/* Large batches are processed in passes of whole images: the forward's input
 * copy is addressed with 32-bit byte offsets (at most 0xF0000000 bytes per
 * pass), the backward keeps at most 1.5 GiB of column gradient (and as much of
 * columns) at a time.  This lowers the two limits for the whole process (0
 * restores a default; values above the defaults are clipped): a knob for memory
 * constrained callers and for tests of the pass loops.  The two values are
 * atomic: a call that runs while another thread changes them uses the old or
 * the new value, never a mixture.  Workspace sizes depend on them and must be
 * queried again after a change; a caller that changes the limits between
 * sizing a workspace and using it gets MDCN_ERR_WORKSPACE at worst.  (No
 * counterpart in the reference, whose im2col_step plays this role for DCNv1.) */
void mdcn_set_pass_limits(uint64_t forward_bytes, uint64_t backward_bytes);

/* Static text for a status code. */
const char *mdcn_status_string(int status);

/* Output height/width for the shape in *p; returns MDCN_OK or MDCN_ERR_SHAPE. */
int mdcn_output_size(const mdcn_params *p, int32_t *Ho, int32_t *Wo);

/* 1 when the fused MFMA kernel covers the shape/dtype in *p, else 0.  Of the
 * pointer fields only `input` is looked at, and only with input_nhwc = 1: a
 * channels-last input is read in place, so it must be 16-byte aligned -- set it
 * before this query and before mdcn_workspace_bytes(). */
int mdcn_fused_eligible(const mdcn_params *p);

/* Which device kernels mdcn_forward() launches for the main stage of the call described by *p (shape,
 * dtype, path, no_k_split; of the pointers only `input` and `output` are looked at, for their alignment):
 * a static string such as "fused3_kernel", "fused3_kernel+fused2_kernel", "fused2_kernel", "fused_kernel",
 * "direct_kernel", "f64_forward_kernel"; "" for an invalid *p.  The first name is the kernel that does
 * most of the work.  For reports and tests (no counterpart in the reference). */
const char *mdcn_forward_kernels(const mdcn_params *p);

/* Bytes of device scratch mdcn_forward() asks for (of the pointer fields only
 * `input` is looked at, see mdcn_fused_eligible()).  The fused path keeps a
 * zero-bordered channels-last copy of the input and the repacked weights there;
 * the direct path and MDCN_F64 need none.  Where the schedule of a launch ends in a
 * round that fills at most half of an XCD's workgroups (see no_k_split), the figure
 * ends with an optional region (one 128 x 256 fp32 tile and a counter per workgroup,
 * 32 MiB on a 256-CU device) through which the workgroups that would otherwise idle
 * share the K range of that round's tiles: a workspace that is smaller by that region
 * is accepted too and only runs that last round unshared.  Returns 0 for an invalid *p
 * (mdcn_forward then reports the error). */
size_t mdcn_workspace_bytes(const mdcn_params *p);

/* Enqueue the forward on `hip_stream` (a hipStream_t; NULL = the null stream).
 * Returns an mdcn_status.  Replaces the body of
 * modulated_deform_conv_forward_fallthrough for device tensors
 * (mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:62-138). */
int mdcn_forward(const mdcn_params *p, void *hip_stream);

/* mdcn_forward() for callers that cannot allocate device memory and have no
 * workspace to pass: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  (No counterpart in the reference, which
 * allocates its columns buffer inside the op.)  `workspace` and
 * `workspace_bytes` of *p are ignored: the input copy and the packed weights go
 * to a buffer of MDCN_NOALLOC_SCRATCH_BYTES that is part of the library's
 * device image (each device the library runs on holds one until the process
 * ends).  Calls whose mdcn_workspace_bytes() exceeds that size return
 * MDCN_ERR_SCRATCH_LIMIT and enqueue nothing (the optional region at the end
 * of the workspace is used when it fits as well and left out otherwise).  The call allocates and frees
 * nothing, on the host or on the device -- from the second call on a device on: the
 * first one asks the runtime for the buffer's address and the device's CU count, so
 * make one call outside a graph capture before capturing.  All calls on one device share the
 * buffer: calls that overlap in time on one device (different streams or
 * threads) race; calls on one stream are ordered by the stream.  Nothing in the
 * buffer has to survive between calls: each call rewrites every byte it reads. */
#define MDCN_NOALLOC_SCRATCH_BYTES (64u << 20)
int mdcn_forward_noalloc(const mdcn_params *p, void *hip_stream);

/* Same work as mdcn_forward(), with HIP events recorded on `hip_stream` around
 * each stage; waits for the stream and reports milliseconds per stage:
 *   ms[0] input re-layout, ms[1] weight repack, ms[2] main kernel, ms[3] total.
 * Stages a path does not run report 0.  For measurement only. */
int mdcn_forward_timed(const mdcn_params *p, void *hip_stream, float ms[4]);

/*
 * The deformable convolution together with the step in front of it in
 * ModulatedDeformConv2dPack.forward (mmcv/ops/modulated_deform_conv.py:327-335):
 *
 *   raw    = conv_offset(x)                 plain conv, Cin -> 3*dgroups*kh*kw channels,
 *                                           kernel/stride/padding/dilation of the DCN (:297-305)
 *   o1, o2, m = chunk(raw, 3, dim=1);  offset = cat(o1, o2);  mask = sigmoid(m)
 *   y      = modulated_deform_conv2d(x, offset, mask, weight, bias, ...)
 *
 * `conv` describes the deformable convolution as for mdcn_forward(); its
 * `offset` and `mask` fields are not read.  The offsets are channels
 * [0, 2*dgroups*kh*kw) of raw as they lie and the mask is the sigmoid of the
 * remaining channels, taken while the kernel reads them, so chunk, cat and
 * sigmoid cost no pass over memory.  Two modes:
 *   offset_weight != NULL: conv_offset runs here as well, on the re-laid-out
 *       input copy the main kernel uses.  offset_weight is
 *       (3*dgroups*kh*kw, Cin, kh, kw), offset_bias (3*dgroups*kh*kw) or NULL.
 *       `raw`, when not NULL, receives the conv_offset output, dense
 *       (N, 3*dgroups*kh*kw, Ho, Wo); NULL keeps it in the workspace only.
 *   offset_weight == NULL: `raw` is an input, the dense conv_offset output
 *       computed by the caller.
 * raw is rounded to `dtype` before it is used and so is the sigmoid, as in the
 * reference's sequence of tensor operations.
 */
typedef struct mdcn_pack_params {
  mdcn_params conv;
  const void *offset_weight;
  const void *offset_bias;
  void *raw;
  int32_t unmodulated;  /* 1: DeformConv2dPack.forward (mmcv/ops/deform_conv.py:405-409): conv_offset has
                           2*dgroups*kh*kw channels, all of them offsets, and there is no mask */
} mdcn_pack_params;

/* Bytes of device scratch mdcn_pack_forward() needs (conv.workspace must hold
 * that many); 0 for an invalid *p. */
size_t mdcn_pack_workspace_bytes(const mdcn_pack_params *p);

/* Enqueue the pack-level forward on `hip_stream`.  Returns an mdcn_status. */
int mdcn_pack_forward(const mdcn_pack_params *p, void *hip_stream);

/* mdcn_pack_forward() with per-stage times: ms[0] input re-layout, ms[1] weight
 * repacks, ms[2] main kernel, ms[3] total, ms[4] conv_offset.  For measurement only. */
int mdcn_pack_forward_timed(const mdcn_pack_params *p, void *hip_stream, float ms[5]);

/*
 * Backward of mdcn_forward(): replaces the body of
 * modulated_deform_conv_backward_fallthrough for device tensors
 * (mmcv/ops/csrc/pytorch/modulated_deform_conv.cpp:140-251) and, with
 * conv.mask == NULL, of deform_conv_backward_input / _parameters
 * (mmcv/ops/csrc/pytorch/deform_conv.cpp:262-525).  `conv` holds the forward's
 * input, offset, mask, weight and geometry (bias and output are not read);
 * grad_output is (N, Cout, Ho, Wo).  Every gradient that is not NULL is written
 * in full (not accumulated into): grad_input like input, grad_offset like
 * offset, grad_mask like mask (must be NULL when conv.mask is), grad_weight like
 * weight, grad_bias (Cout).  grad_input and grad_offset/grad_mask are produced
 * together: pass all of them or none.  Sums are formed in fp32 and rounded once.
 * The scatter into grad_input (and, for shapes off the matrix-core path, the
 * pixel reduction of grad_weight) uses floating-point atomics, so results vary
 * in the last bits from run to run, as the reference's CUDA kernels' do.
 */
typedef struct mdcn_bwd_params {
  mdcn_params conv;
  const void *grad_output;
  void *grad_input;
  void *grad_offset;
  void *grad_mask;
  void *grad_weight;
  void *grad_bias;
} mdcn_bwd_params;

/* Bytes of device scratch mdcn_backward() needs for *p as it will be passed to
 * mdcn_backward() (gradient pointers set: which gradients are asked for decides
 * what is staged): fp32 staging of grad_input and grad_weight for 16-bit
 * tensors and, for shapes whose column gradient runs on the matrix cores,
 * pixel-major copies of input and grad_output, the transposed weights and the
 * column gradient of up to 1.5 GiB of images at a time; may be 0.
 * conv.path: MDCN_PATH_AUTO picks by shape and size; MDCN_PATH_FUSED asks for
 * the tiled kernels whatever the problem size (MDCN_ERR_PATH if the shape rules
 * them out); MDCN_PATH_DIRECT keeps the one-workgroup-per-tap kernel. */
size_t mdcn_backward_workspace_bytes(const mdcn_bwd_params *p);

/* Enqueue the backward on `hip_stream`.  Returns an mdcn_status. */
int mdcn_backward(const mdcn_bwd_params *p, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* MDCN_H_ */
