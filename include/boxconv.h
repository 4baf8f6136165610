/* libboxconv_hip.so -- box convolution (integral-image box filters) for AMD gfx950 (MI355X).
 *
 * C ABI: plain pointers and sizes, no torch types. Every pointer is DEVICE memory on the current
 * HIP device unless stated otherwise; the caller owns every buffer, including scratch. `stream`
 * is a hipStream_t passed as void* (NULL = the null stream). All work is enqueued on that stream
 * and the call returns without synchronising. Nothing here allocates device memory.
 *
 * Return value: 0 on success; a positive value is a hipError_t from a launch; negative values are
 * BOXCONV_E_* argument errors detected before anything was launched. boxconv_last_error() gives
 * the message of the last failure on the calling thread.
 *
 * The four entry-point families replace the four functions of the reference's native module
 * `box_convolution_cpp_cuda` (reference src/bind.cpp:29-34); _f32 / _f64 select the element type
 * (the reference dispatches on the tensor dtype).
 *
 * Layouts (all contiguous, row-major):
 *   input            [batch, in_planes, h, w]
 *   input_integrated [batch, in_planes, h+1, w+1]     row 0 and column 0 are zero
 *   x_min .. y_max   [in_planes, num_filters]         REAL pixel units (already multiplied by the
 *                                                     module's reparametrization factors);
 *                                                     x_* are ROW bounds, y_* COLUMN bounds
 *   output, grad_output [batch, in_planes*num_filters, h, w]   channel index = plane*num_filters + filter
 */
#ifndef BOXCONV_H_
#define BOXCONV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BOXCONV_ABI_VERSION 4

#define BOXCONV_E_INVALID_ARGUMENT (-1) /* null pointer, non-positive size, ... */
#define BOXCONV_E_WORKSPACE        (-2) /* workspace missing or smaller than *_workspace_bytes() */
#define BOXCONV_E_TOO_LARGE        (-3) /* a tensor has 2^31 or more elements */

int boxconv_abi_version(void);

/* Message of the last error on this thread ("" if none). Never NULL; valid until the next call
 * on this thread. */
const char* boxconv_last_error(void);

/* The library's measurement and test switches (environment variables BOXCONV_*, listed in the
 * integration notes) are read once, at the first call that needs them; no entry point calls getenv
 * on its way to a launch. boxconv_reload_env() reads them again, for a test that changes one
 * inside a running process. Not synchronised with calls in flight on other threads. No
 * counterpart in the reference. */
void boxconv_reload_env(void);

/* ---- per-kernel timing (measurement aid; no counterpart in the reference) ---------------------
 * boxconv_profile_arm(name): from now on every launch of the kernel called `name` is bracketed by
 * a pair of HIP events recorded on the stream it is launched on (so the time is that kernel's
 * alone, whatever else the entry point launches). Names: "band_colsum", "band_prefix",
 * "band_scan", "forward_rows", "grad_output_stream", "grad_input_cols",
 * "param_grad_finalize", "fill_zero", "fill_marker", "clip", "forward_gather", "grad_input_gather",
 * "int_row_prefix", "int_col_prefix", "probe_copy_bands", "probe_grad_input_pattern",
 * "grad_params_gather".
 * NULL or "" disarms. Arming discards earlier measurements.
 * boxconv_profile_arm_every(name, n): the same, but only every n-th launch of that kernel (the
 * first, the (n+1)-th, ...) is bracketed; an event pair costs a few microseconds of GPU time, which
 * a caller that also times the whole run may not want to pay at every launch.
 * boxconv_profile_collect(&total_ms, &launches): waits for the recorded events, returns the summed
 * kernel time and the number of launches, then disarms. Process-wide state; meant for benchmarks. */
int boxconv_profile_arm(const char* kernel_name);
int boxconv_profile_arm_every(const char* kernel_name, int every);
int boxconv_profile_collect(double* total_ms, int* launches);

/* A plain copy with the access pattern of the backward's streaming pass over grad_output
 * (measurement aid; no counterpart in the reference): `planes` planes of h x w floats are copied
 * into planes of (h+1) x w floats (rows 1..h; row 0 is not touched), a workgroup of w/4 lanes
 * streaming `rows_per_group` consecutive rows, 16 bytes per lane and row, `rows_in_flight` (2, 4
 * or 8) rows loaded before they are stored, non-temporal stores. Its rate is what the memory
 * system gives a kernel that reads and writes with that pattern, the yardstick the benchmark
 * prints beside the kernels' own rates. w a multiple of 256 up to 4096, h a multiple of
 * rows_per_group, rows_per_group a multiple of rows_in_flight. */
int boxconv_probe_copy_bands(const float* src, float* dst, int64_t planes, int h, int w,
                             int rows_per_group, int rows_in_flight, void* stream);

/* The loads and stores of the backward's grad-input pass without its arithmetic (measurement aid;
 * no counterpart in the reference), for rows of 1024 floats: column_workspace holds
 * planes * num_filters planes of (h+1) x 1024 floats, out planes of h x 1024. A workgroup owns 8
 * output rows i0.. of a plane and reads, per filter f of input plane c = plane % in_planes, the 9
 * rows from i0 + x_lo[c*F+f] - 1 and the 9 rows from i0 + x_hi[c*F+f] (clamped to [0, h]) of that
 * filter's plane, 16 bytes per lane and row, as the kernel does. mode 0: both runs; 1: the second
 * run only (every row is then read once); 2: the first run from a few MB that stay in the L2
 * (what the second read of a row costs when it always hits). h a multiple of 8. */
int boxconv_probe_grad_input_pattern(const float* column_workspace, float* out, const int* x_lo,
                                     const int* x_hi, int64_t planes, int in_planes, int num_filters, int h,
                                     int mode, void* stream);

/* ---- integral image ------------------------------------------------------------------------
 * Replaces `integral_image(Tensor) -> Tensor`, reference src/integral_image_interface.cpp:8-27
 * (kernels: src/integral_image.cpp:8-39). `planes` is the product of all leading dimensions.
 * out[p][r+1][c+1] = sum_{i<=r, j<=c} in[p][i][j]; out[p][0][*] = out[p][*][0] = 0.
 * workspace: boxconv_integral_image_workspace_bytes(planes, h, w) bytes, 8-byte aligned (may be
 * NULL when that size is 0). */
size_t boxconv_integral_image_workspace_bytes(int64_t planes, int h, int w);
int boxconv_integral_image_f32(const float* in, float* out, int64_t planes, int h, int w,
                               void* workspace, size_t workspace_bytes, void* stream);
int boxconv_integral_image_f64(const double* in, double* out, int64_t planes, int h, int w,
                               void* workspace, size_t workspace_bytes, void* stream);

/* Integral image of an integer tensor. The reference's function takes every ATen type
 * (AT_DISPATCH_ALL_TYPES, src/integral_image.cpp:14; wrapper src/integral_image_interface.cpp:8-27):
 * the row sum runs in int64 and every entry is stored in the tensor's own type, so out holds the
 * exact sums modulo 2^bits (src/integral_image.cpp:20-37). `dtype` selects the element type of
 * both tensors. No workspace. Not used by BoxConv2d; two plain launches, not tuned. */
#define BOXCONV_U8  16 /* uint8_t */
#define BOXCONV_I8  17 /* int8_t */
#define BOXCONV_I16 18 /* int16_t */
#define BOXCONV_I32 19 /* int32_t */
#define BOXCONV_I64 20 /* int64_t */
int boxconv_integral_image_int(const void* in, void* out, int dtype, int64_t planes, int h, int w,
                               void* stream);

/* The same integral image for callers that cannot allocate or pass a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in
 * the reference. Same kernels and bit-identical results as boxconv_integral_image_f32; the band
 * column sums go to an array of BOXCONV_STATIC_SCRATCH_BYTES bytes that the library holds in the
 * memory of every GPU it is loaded on until the process ends. The call allocates and frees
 * nothing (the first call on a device looks the array's address up once; make that call before
 * starting a graph capture).
 * Shapes with boxconv_integral_image_workspace_bytes(planes, h, w) > BOXCONV_STATIC_SCRATCH_BYTES
 * are refused with BOXCONV_E_TOO_LARGE (the headline shape, 32 planes of 512 x 1024, needs 3.75 MiB).
 * All calls on one GPU share the one array: two calls that overlap in time on the same GPU (two
 * streams, two threads) race; calls on one stream are ordered and safe. */
#define BOXCONV_STATIC_SCRATCH_BYTES (8u << 20)
int boxconv_integral_image_static_f32(const float* in, float* out, int64_t planes, int h, int w,
                                      void* stream);

/* Element type codes of the entry points that read or write half precision. */
#define BOXCONV_F32 0
#define BOXCONV_F16 1  /* IEEE binary16 */
#define BOXCONV_BF16 2 /* bfloat16 */

/* float32 integral image of a float16 / bfloat16 input (input_dtype: BOXCONV_F16 or BOXCONV_BF16),
 * sums carried in double as for float input. The reference integrates a half-precision tensor in
 * half precision (src/integral_image_cuda.cu:67-173, AT_DISPATCH_FLOATING_TYPES_AND_HALF), which
 * overflows at 65504; this is what the inference entry point below is fed instead. Rows of at
 * most 2048 columns (BOXCONV_E_TOO_LARGE otherwise: convert to float first). Same workspace as
 * boxconv_integral_image_f32. */
int boxconv_integral_image_half_f32(const void* in, int input_dtype, float* out, int64_t planes,
                                    int h, int w, void* workspace, size_t workspace_bytes,
                                    void* stream);

/* ---- forward ----------------------------------------------------------------------------------
 * Replaces `box_convolution_forward(input_integrated, x_min, x_max, y_min, y_max, normalize,
 * exact) -> Tensor[B, C*F, h, w]`, reference src/box_convolution_interface.cpp:13-139 (kernels:
 * src/box_convolution.cpp:14-40, 100-261, 765-793). normalize: divide by the box area;
 * exact = 0: bounds are rounded towards the smaller box first. */
int boxconv_forward_f32(const float* input_integrated, const float* x_min, const float* x_max,
                        const float* y_min, const float* y_max, float* output, int batch,
                        int in_planes, int num_filters, int h, int w, int normalize, int exact,
                        void* stream);
int boxconv_forward_f64(const double* input_integrated, const double* x_min, const double* x_max,
                        const double* y_min, const double* y_max, double* output, int batch,
                        int in_planes, int num_filters, int h, int w, int normalize, int exact,
                        void* stream);

/* ---- training-mode forward in one call -------------------------------------------------------
 * What `BoxConv2d.forward` does when `self.training` (reference
 * box_convolution/box_convolution_module.py:203-214 and box_convolution_function.py:41-46):
 * clip_parameters on the stored bounds (in place), stored -> real units, integral_image,
 * box_convolution_forward. Same results as boxconv_clip_reparametrize_*, boxconv_integral_image_*
 * and boxconv_forward_* called in turn, with one launch fewer (the clip shares the launch that
 * prepares the integral image's workspace).
 * x_min..y_max: [in_planes*num_filters], stored units, clipped in place. real_parameters:
 * [4][in_planes*num_filters] out (x_min, x_max, y_min, y_max in pixel units). input_integrated:
 * [batch, in_planes, h+1, w+1] out. output: [batch, in_planes*num_filters, h, w] out.
 * workspace: boxconv_integral_image_workspace_bytes(batch*in_planes, h, w) bytes, 8-byte aligned. */
int boxconv_training_forward_f32(const float* input, float* x_min, float* x_max, float* y_min,
                                 float* y_max, float* real_parameters, float* input_integrated,
                                 float* output, int batch, int in_planes, int num_filters, int h,
                                 int w, double reparametrization_h, double reparametrization_w,
                                 double max_input_h, double max_input_w, int normalize, int exact,
                                 void* workspace, size_t workspace_bytes, void* stream);
int boxconv_training_forward_f64(const double* input, double* x_min, double* x_max, double* y_min,
                                 double* y_max, double* real_parameters, double* input_integrated,
                                 double* output, int batch, int in_planes, int num_filters, int h,
                                 int w, double reparametrization_h, double reparametrization_w,
                                 double max_input_h, double max_input_w, int normalize, int exact,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* ---- eval-mode forward in one call --------------------------------------------------------------
 * What `BoxConv2d.forward` does when `self.training` is false (reference
 * box_convolution/box_convolution_module.py:208-214 and box_convolution_function.py:41-46): no
 * clipping; stored -> real units, integral_image, box_convolution_forward. The stored bounds are
 * only read. Same results as `stored * reparametrization`, boxconv_integral_image_* and
 * boxconv_forward_* in turn; arguments as for boxconv_training_forward_* without the clip limits. */
int boxconv_inference_forward_f32(const float* input, const float* x_min, const float* x_max,
                                  const float* y_min, const float* y_max, float* real_parameters,
                                  float* input_integrated, float* output, int batch, int in_planes,
                                  int num_filters, int h, int w, double reparametrization_h,
                                  double reparametrization_w, int normalize, int exact, void* workspace,
                                  size_t workspace_bytes, void* stream);
int boxconv_inference_forward_f64(const double* input, const double* x_min, const double* x_max,
                                  const double* y_min, const double* y_max, double* real_parameters,
                                  double* input_integrated, double* output, int batch, int in_planes,
                                  int num_filters, int h, int w, double reparametrization_h,
                                  double reparametrization_w, int normalize, int exact, void* workspace,
                                  size_t workspace_bytes, void* stream);

/* ---- training- and eval-mode forward in one call, half-precision tensors -------------------------
 * The two entry points above for a float16 / bfloat16 input and output (io_dtype: BOXCONV_F16 or
 * BOXCONV_BF16, both tensors of that type) with float32 parameters: what the reference's
 * `BoxConv2d.forward` (box_convolution/box_convolution_module.py:208-214) does with a half tensor
 * on its CUDA path, except that the integral image (input_integrated, float32 out, what
 * boxconv_backward_half_f32 takes) and all sums are float32 / double, as in
 * boxconv_integral_image_half_f32 and boxconv_forward_fused_f32, whose results this call returns
 * bit for bit. clip != 0: training mode (the stored parameters are projected in place first, limits
 * max_input_h / max_input_w); clip == 0: eval mode (the stored parameters are only read).
 * Rows of at most 2048 columns (BOXCONV_E_TOO_LARGE otherwise: convert to float first). */
int boxconv_training_forward_half_f32(const void* input, int io_dtype, float* x_min, float* x_max,
                                      float* y_min, float* y_max, float* real_parameters,
                                      float* input_integrated, void* output, int batch, int in_planes,
                                      int num_filters, int h, int w, double reparametrization_h,
                                      double reparametrization_w, double max_input_h, double max_input_w,
                                      int clip, int normalize, int exact, void* workspace,
                                      size_t workspace_bytes, void* stream);

/* ---- forward, half-precision output and fused tail (inference) ------------------------------
 * The same box sums as boxconv_forward_f32 (reference src/box_convolution_interface.cpp:13-139),
 * computed in float from a float integral image, with what a network does to them next folded
 * into the store: the tail of the reference's BottleneckBoxConv block in eval mode, BoxConv2d ->
 * BatchNorm2d -> Dropout2d (identity) -> residual add -> ReLU
 * (examples/Cityscapes/models/ENet.py:290-304):
 *     y = S * channel_scale[c*F+f] + channel_shift[c*F+f] + residual[b][c*F+f][i][j]
 *     output = relu ? max(y, 0) : y,  rounded to nearest even into the output type.
 * output_dtype: BOXCONV_F32, BOXCONV_F16 (IEEE binary16) or BOXCONV_BF16; `output` and `residual`
 * point at elements of that type, [batch, in_planes*num_filters, h, w]. channel_scale and
 * channel_shift are float [in_planes*num_filters] (an eval-mode BatchNorm folds to
 * scale = gamma / sqrt(var + eps), shift = beta - mean * scale). residual, channel_scale and
 * channel_shift may each be NULL (no residual, scale 1, shift 0). There is no backward for
 * this entry point. */
int boxconv_forward_fused_f32(const float* input_integrated, const float* x_min,
                              const float* x_max, const float* y_min, const float* y_max,
                              void* output, int output_dtype, const void* residual,
                              const float* channel_scale, const float* channel_shift, int relu,
                              int batch, int in_planes, int num_filters, int h, int w,
                              int normalize, int exact, void* stream);

/* ---- backward ---------------------------------------------------------------------------------
 * Replaces `box_convolution_backward(input_integrated, x_min, x_max, y_min, y_max, grad_output,
 * output, reparametrization_h, reparametrization_w, normalize, exact, input_needs_grad,
 * x_min_needs_grad, x_max_needs_grad, y_min_needs_grad, y_max_needs_grad) -> 5 Tensors`,
 * reference src/box_convolution_interface.cpp:141-395 (kernels: src/box_convolution.cpp:43-98,
 * 286-715). A gradient is wanted iff its output pointer is non-NULL:
 *   grad_input [batch, in_planes, h, w];  grad_x_min .. grad_y_max [in_planes, num_filters],
 * the latter already multiplied by reparametrization_h (x) / reparametrization_w (y).
 * `output` (the saved forward result) is accepted for signature parity and may be NULL: the
 * normalisation term sum(grad_output*output) is recomputed from input_integrated instead of
 * re-reading it.
 * workspace: boxconv_backward_workspace_bytes(...) bytes, 256-byte aligned. It receives the
 * backward's one intermediate per (plane, filter) - h+1 rows of grad_output filtered along the
 * row and summed down the rows of a band (the bulk; for rows wider than 4096 columns, 2048 in
 * float64, a true integral image of grad_output instead) - and the per-box accumulators. */
size_t boxconv_backward_workspace_bytes(int batch, int in_planes, int num_filters, int h, int w,
                                        int elem_size, int input_needs_grad,
                                        int params_need_grad);
int boxconv_backward_f32(const float* input_integrated, const float* x_min, const float* x_max,
                         const float* y_min, const float* y_max, const float* grad_output,
                         const float* output, float reparametrization_h,
                         float reparametrization_w, int normalize, int exact, float* grad_input,
                         float* grad_x_min, float* grad_x_max, float* grad_y_min,
                         float* grad_y_max, int batch, int in_planes, int num_filters, int h,
                         int w, void* workspace, size_t workspace_bytes, void* stream);
int boxconv_backward_f64(const double* input_integrated, const double* x_min, const double* x_max,
                         const double* y_min, const double* y_max, const double* grad_output,
                         const double* output, float reparametrization_h,
                         float reparametrization_w, int normalize, int exact, double* grad_input,
                         double* grad_x_min, double* grad_x_max, double* grad_y_min,
                         double* grad_y_max, int batch, int in_planes, int num_filters, int h,
                         int w, void* workspace, size_t workspace_bytes, void* stream);

/* The same backward pass with grad_output and grad_input in half precision (io_dtype: BOXCONV_F16
 * or BOXCONV_BF16; both tensors of that type), everything else float: the float32 integral image
 * of the input as saved by the forward, float32 box bounds, float32 parameter gradients, float32
 * (and double) sums. The reference dispatches its CUDA kernels on half tensors
 * (src/box_convolution_cuda_backward.cu:176,431, AT_DISPATCH_FLOATING_TYPES_AND_HALF) and then
 * integrates grad_output in half precision; here its rows are widened to float as they are read
 * and grad_input is rounded once, in the store. Same workspace as boxconv_backward_f32
 * (boxconv_backward_workspace_bytes with elem_size 4). Rows of at most 4096 columns
 * (BOXCONV_E_TOO_LARGE otherwise: convert to float first). */
int boxconv_backward_half_f32(const float* input_integrated, const float* x_min, const float* x_max,
                              const float* y_min, const float* y_max, const void* grad_output,
                              int io_dtype, float reparametrization_h, float reparametrization_w,
                              int normalize, int exact, void* grad_input, float* grad_x_min,
                              float* grad_x_max, float* grad_y_min, float* grad_y_max, int batch,
                              int in_planes, int num_filters, int h, int w, void* workspace,
                              size_t workspace_bytes, void* stream);

/* ---- clip parameters --------------------------------------------------------------------------
 * Replaces `clip_parameters(x_min, x_max, y_min, y_max, reparametrization_h, reparametrization_w,
 * max_input_h, max_input_w, exact) -> None`, reference src/box_convolution_interface.cpp:397-415
 * (kernel: src/box_convolution.cpp:729-763). In place on the STORED (reparametrized) parameters,
 * n = in_planes*num_filters elements each. */
int boxconv_clip_parameters_f32(float* x_min, float* x_max, float* y_min, float* y_max, int n,
                                double reparametrization_h, double reparametrization_w,
                                double max_input_h, double max_input_w, int exact, void* stream);
int boxconv_clip_parameters_f64(double* x_min, double* x_max, double* y_min, double* y_max, int n,
                                double reparametrization_h, double reparametrization_w,
                                double max_input_h, double max_input_w, int exact, void* stream);

/* ---- clip + stored -> real units in one launch ------------------------------------------------
 * What a training-mode forward of the reference does with the parameters before anything else:
 * `clip_parameters(...)` (as above; reference box_convolution/box_convolution_module.py:203-206)
 * followed by `reparametrize(..., inverse=True)` (reference
 * box_convolution/box_convolution_function.py:5-27, called at :41-43), i.e. four more element-wise
 * multiplications. The stored parameters are clipped in place exactly as by
 * boxconv_clip_parameters_*; real_parameters ([4][n]: x_min, x_max, y_min, y_max) receives
 * clipped * reparametrization, the factor rounded to the element type first (a tensor times a
 * Python float). */
int boxconv_clip_reparametrize_f32(float* x_min, float* x_max, float* y_min, float* y_max,
                                   float* real_parameters, int n, double reparametrization_h,
                                   double reparametrization_w, double max_input_h,
                                   double max_input_w, int exact, void* stream);
int boxconv_clip_reparametrize_f64(double* x_min, double* x_max, double* y_min, double* y_max,
                                   double* real_parameters, int n, double reparametrization_h,
                                   double reparametrization_w, double max_input_h,
                                   double max_input_w, int exact, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* BOXCONV_H_ */
