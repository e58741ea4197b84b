/*
 * C ABI of the MI355X (gfx950) ROIAlign launcher library, libmobula_hip.so.
 *
 * The first two functions are, name for name and argument for argument, what
 * the reference's Python binding resolves with ctypes for the float
 * instantiation of its ROIAlign kernels:
 *   - symbol name  <func>_<md5(argument C type list)[:8]>   mobula/func.py:13-50
 *   - signature    (device_id, kernel arguments...)          mobula/op/templates/kernel_code.cpp:1-5
 *   - kernel arguments                                       opzoo/ROIAlign/ROIAlign.cpp:10-16, 79-83
 *   - call site    func(dev_id, *raw_pointers)               mobula/func.py:155-156
 *
 * Conventions (all entry points):
 *   device_id >= 0  every pointer is device memory of that GPU; the launch
 *                   goes to the stream set with mobula_hip_set_stream() on the
 *                   calling thread (default: the null stream, and the call
 *                   returns only when the result is complete, like the
 *                   reference, context/hip_ctx.h:62-93).
 *   device_id == -1 every pointer is host memory; the library stages the
 *                   buffers through GPU memory and returns when the result is
 *                   in the host buffers.  There is no CPU implementation.
 *   Tensors are dense: data/bottom_diff NCHW [N,C,H,W], rois [R,5] rows
 *   [batch_idx, x1, y1, x2, y2], top [R,C,PH,PW]; R = nthreads/(C*PH*PW).
 *   N is not an argument of the reference ABI: it is taken from the element
 *   count declared with mobula_hip_set_arg_extents(), else read back from the
 *   largest batch index (one blocking copy).
 *   No return codes: a failed call leaves a message for
 *   mobula_hip_last_error() and does not terminate the process (the reference
 *   prints and calls exit(-1), mobula/cpp/include/logging.h:23-26).
 */
#ifndef MOBULA_ROIALIGN_H_
#define MOBULA_ROIALIGN_H_

#ifdef __cplusplus
extern "C" {
#endif

/* top_data[r,c,ph,pw] = mean over the sampling grid of bilinear samples.
 * Replaces: roi_align_forward_kernel<float>, opzoo/ROIAlign/ROIAlign.cpp:9-76. */
void roi_align_forward_ab78de3c(const int device_id, const int nthreads,
                                const float* bottom_data, const float spatial_scale,
                                const int channels, const int height, const int width,
                                const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const float* bottom_rois,
                                float* top_data);

/* bottom_diff += scatter of top_diff (accumulates; the caller zeroes).
 * Replaces: roi_align_backward_kernel<float>, opzoo/ROIAlign/ROIAlign.cpp:78-161.
 * Note the argument order: bottom_diff before bottom_rois. */
void roi_align_backward_f318a24e(const int device_id, const int nthreads, const float* top_diff,
                                 const float spatial_scale, const int channels, const int height,
                                 const int width, const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, float* bottom_diff,
                                 const float* bottom_rois);

/* The reference's <double> instantiation of the forward (same kernel template,
 * T = double: map, boxes, scale and result in binary64).
 * Replaces: roi_align_forward_kernel<double>, opzoo/ROIAlign/ROIAlign.cpp:9-76
 * under the name mobula/func.py:13-50 derives for it. */
void roi_align_forward_6b9e6c9b(const int device_id, const int nthreads, const double* bottom_data,
                                const double spatial_scale, const int channels, const int height,
                                const int width, const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const double* bottom_rois, double* top_data);

/* Makes device_id the current device.
 * Replaces: set_device, mobula/cpp/include/context/context.h:15-17. */
void set_device(const int device_id);

/* ---- Extensions: no counterpart in the reference ------------------------ */

/* bottom_diff = scatter of top_diff: overwrites all N*C*H*W elements (zero
 * where no ROI contributes).  Fuses the operator's zero-fill
 * (opzoo/ROIAlign/ROIAlign.py:33-34) with the scatter. */
void roi_align_backward_assign_a8793cbe(const int device_id, const int nthreads,
                                        const float* top_diff, const float spatial_scale,
                                        const int channels, const int height, const int width,
                                        const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        float* bottom_diff, const float* bottom_rois);

/* The forward pass for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same result as roi_align_forward_ab78de3c
 * (same kernels); the scratch memory those kernels need (the channel-blocked
 * copy of the map and the ROI order) is a fixed buffer of 48 MiB that every GPU
 * the library runs on holds until the process ends, so the call makes no
 * allocation, no stream and no event.  num_images is the N of the [N,C,H,W]
 * map.  Device memory only.  A problem that needs more scratch than the buffer
 * holds (about N*C*H*W*4 + R*4 bytes) is refused with an error.  All calls on
 * one GPU share the buffer: calls that overlap in time on one GPU race. */
void roi_align_forward_noalloc_83212f20(const int device_id, const int nthreads,
                                        const float* bottom_data, const float spatial_scale,
                                        const int channels, const int height, const int width,
                                        const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        const float* bottom_rois, float* top_data);
/* Looks up the fixed buffer's address on device_id ahead of the first call
 * there (which does it otherwise); returns the buffer's size in bytes, -1 on error. */
long long mobula_hip_roialign_noalloc_init(const int device_id);

/* Backward in binary64, accumulating and overwriting.  The names are what the
 * reference's scheme gives the <double> instantiations, but the reference cannot
 * build them: its atomic_add takes float only
 * (mobula/cpp/include/context/cpu_ctx.h:37, context/hip_ctx.h:108-114). */
void roi_align_backward_2b6c6dfa(const int device_id, const int nthreads, const double* top_diff,
                                 const double spatial_scale, const int channels, const int height,
                                 const int width, const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, double* bottom_diff, const double* bottom_rois);
void roi_align_backward_assign_4620f85e(const int device_id, const int nthreads, const double* top_diff,
                                        const double spatial_scale, const int channels, const int height,
                                        const int width, const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        double* bottom_diff, const double* bottom_rois);

/* Forward with IEEE binary16 storage of bottom_data / top_data (passed as
 * 16-bit patterns), fp32 rois and fp32 accumulation. */
void roi_align_forward_e874c59a(const int device_id, const int nthreads,
                                const unsigned short* bottom_data, const float spatial_scale,
                                const int channels, const int height, const int width,
                                const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const float* bottom_rois,
                                unsigned short* top_data);

/* Backward with binary16 top_diff / bottom_diff (fp32 rois; sums are formed in
 * fp32 and rounded once per element).  The reference has float atomics only
 * (context/cpu_ctx.h:37-62), hence no counterpart. */
void roi_align_backward_23175303(const int device_id, const int nthreads, const unsigned short* top_diff,
                                 const float spatial_scale, const int channels, const int height,
                                 const int width, const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, unsigned short* bottom_diff,
                                 const float* bottom_rois);
void roi_align_backward_assign_7924dbc8(const int device_id, const int nthreads,
                                        const unsigned short* top_diff, const float spatial_scale,
                                        const int channels, const int height, const int width,
                                        const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        unsigned short* bottom_diff, const float* bottom_rois);

/* The same three with bfloat16 storage (the upper 16 bits of a binary32, passed
 * as unsigned short; fp32 rois, fp32 arithmetic, results rounded to nearest-even). */
void roi_align_forward_f951d439(const int device_id, const int nthreads, const unsigned short* bottom_data,
                                const float spatial_scale, const int channels, const int height,
                                const int width, const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const float* bottom_rois, unsigned short* top_data);
void roi_align_backward_0c43e974(const int device_id, const int nthreads, const unsigned short* top_diff,
                                 const float spatial_scale, const int channels, const int height,
                                 const int width, const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, unsigned short* bottom_diff, const float* bottom_rois);
void roi_align_backward_assign_86156afd(const int device_id, const int nthreads,
                                        const unsigned short* top_diff, const float spatial_scale,
                                        const int channels, const int height, const int width,
                                        const int pooled_height, const int pooled_width,
                                        const int sampling_ratio, const int num_images,
                                        unsigned short* bottom_diff, const float* bottom_rois);

/* The three operations on channels-last tensors: the map as [N,H,W,C], the pooled
 * tensor as [R,PH,PW,C] (what a torch tensor in torch.channels_last format holds);
 * scalar arguments as above (channels, height, width name C, H, W).  No
 * counterpart in the reference, whose binding makes tensors NCHW-contiguous
 * before the call (mobula/func.py:79-92): with these entry points neither that
 * copy nor the library's own re-layout of the map and of top_diff is made.
 * Device pointers only, 16-byte aligned.  A shape the fast kernels do not take is
 * an error (mobula_hip_last_error), not a slow path: ask
 * mobula_hip_roialign_nhwc_supported first and convert to NCHW otherwise.  Takes:
 * forward: channels a multiple of 4 (fp32) or 8 (16-bit types), pooled_width <= 50,
 * one image below 2 GiB; backward: fp32, fp16 or bfloat16, channels a multiple of
 * 4, sampling_ratio <= 64 (an adaptive grid, sampling_ratio <= 0, is taken; a call
 * whose boxes give it more than 2^15 points per bin along an axis, or whose stream
 * is being captured into a graph while sampling_ratio is not 1 or 2, fails with an
 * error: the NCHW entry points take those), pooled_width <= 32, pooled_height <= 32,
 * R * PH * PW * C * 4 below 2 GiB. */
void roi_align_forward_nhwc_ab78de3c(const int device_id, const int nthreads, const float* bottom_data,
                                     const float spatial_scale, const int channels, const int height,
                                     const int width, const int pooled_height, const int pooled_width,
                                     const int sampling_ratio, const float* bottom_rois, float* top_data);
void roi_align_forward_nhwc_e874c59a(const int device_id, const int nthreads,
                                     const unsigned short* bottom_data, const float spatial_scale,
                                     const int channels, const int height, const int width,
                                     const int pooled_height, const int pooled_width,
                                     const int sampling_ratio, const float* bottom_rois,
                                     unsigned short* top_data);
void roi_align_forward_nhwc_f951d439(const int device_id, const int nthreads,   /* bfloat16 storage */
                                     const unsigned short* bottom_data, const float spatial_scale,
                                     const int channels, const int height, const int width,
                                     const int pooled_height, const int pooled_width,
                                     const int sampling_ratio, const float* bottom_rois,
                                     unsigned short* top_data);
void roi_align_backward_nhwc_f318a24e(const int device_id, const int nthreads, const float* top_diff,
                                      const float spatial_scale, const int channels, const int height,
                                      const int width, const int pooled_height, const int pooled_width,
                                      const int sampling_ratio, float* bottom_diff, const float* bottom_rois);
void roi_align_backward_nhwc_assign_a8793cbe(const int device_id, const int nthreads, const float* top_diff,
                                             const float spatial_scale, const int channels, const int height,
                                             const int width, const int pooled_height, const int pooled_width,
                                             const int sampling_ratio, const int num_images, float* bottom_diff,
                                             const float* bottom_rois);
/* The channels-last backward with 16-bit tensors: binary16 (23175303 / 7924dbc8) and
 * bfloat16 (0c43e974 / 86156afd); dy and dx have the same type, sums are fp32. */
void roi_align_backward_nhwc_23175303(const int device_id, const int nthreads, const unsigned short* top_diff,
                                      const float spatial_scale, const int channels, const int height,
                                      const int width, const int pooled_height, const int pooled_width,
                                      const int sampling_ratio, unsigned short* bottom_diff,
                                      const float* bottom_rois);
void roi_align_backward_nhwc_assign_7924dbc8(const int device_id, const int nthreads,
                                             const unsigned short* top_diff, const float spatial_scale,
                                             const int channels, const int height, const int width,
                                             const int pooled_height, const int pooled_width,
                                             const int sampling_ratio, const int num_images,
                                             unsigned short* bottom_diff, const float* bottom_rois);
void roi_align_backward_nhwc_0c43e974(const int device_id, const int nthreads, const unsigned short* top_diff,
                                      const float spatial_scale, const int channels, const int height,
                                      const int width, const int pooled_height, const int pooled_width,
                                      const int sampling_ratio, unsigned short* bottom_diff,
                                      const float* bottom_rois);
void roi_align_backward_nhwc_assign_86156afd(const int device_id, const int nthreads,
                                             const unsigned short* top_diff, const float spatial_scale,
                                             const int channels, const int height, const int width,
                                             const int pooled_height, const int pooled_width,
                                             const int sampling_ratio, const int num_images,
                                             unsigned short* bottom_diff, const float* bottom_rois);
/* 1 if the channels-last entry points take the shape, else 0.  backward != 0 asks
 * about the backward entry points; elem_bytes is 4 (fp32) or 2 (fp16, bfloat16). */
int mobula_hip_roialign_nhwc_supported(int backward, int elem_bytes, int channels, int height, int width,
                                       int pooled_height, int pooled_width, int sampling_ratio,
                                       long long num_rois);

/* ---- Convolution -------------------------------------------------------- */

/* One image: data_col[c, kh, kw, oh, ow] = data_im[c, ih, iw], zero in the
 * padding; n = element count of data_col.
 * Replaces: im2col_kernel<float>, opzoo/Convolution/Convolution.cpp:13-45. */
void im2col_341af5d3(const int device_id, const int n, const float* data_im, const int height,
                     const int width, const int kernel_h, const int kernel_w, const int pad_h,
                     const int pad_w, const int stride_h, const int stride_w, const int dilation_h,
                     const int dilation_w, const int height_col, const int width_col, float* data_col);

/* One image: data_im[c, h, w] = sum of the column entries unfolded from it;
 * n = element count of data_im.
 * Replaces: col2im_kernel<float>, opzoo/Convolution/Convolution.cpp:47-90. */
void col2im_341af5d3(const int device_id, const int n, const float* data_col, const int height,
                     const int width, const int kernel_h, const int kernel_w, const int pad_h,
                     const int pad_w, const int stride_h, const int stride_w, const int dilation_h,
                     const int dilation_w, const int height_col, const int width_col, float* data_im);

/* Extensions: the products the reference operator assembles per image from
 * im2col / col2im and the framework's matrix product
 * (opzoo/Convolution/Convolution.py:17-57), as one call each on the matrix
 * cores.  x [batch, channels, height, width], weight [filters, channels,
 * kernel_h, kernel_w], y / dy [batch, filters, OH, OW]; device memory only.
 * n is the element count of the output tensor; accumulate != 0 adds to it. */
void conv2d_forward_c6a7aa85(const int device_id, const int n, const float* x, const float* weight,
                             const float* bias, const int has_bias, const int batch,
                             const int channels, const int height, const int width, const int filters,
                             const int kernel_h, const int kernel_w, const int pad_h, const int pad_w,
                             const int stride_h, const int stride_w, const int dilation_h,
                             const int dilation_w, float* y);
void conv2d_backward_data_ecf81c91(const int device_id, const int n, const float* dy,
                                   const float* weight, const int accumulate, const int batch,
                                   const int channels, const int height, const int width,
                                   const int filters, const int kernel_h, const int kernel_w,
                                   const int pad_h, const int pad_w, const int stride_h,
                                   const int stride_w, const int dilation_h, const int dilation_w,
                                   float* dx);
/* (With the option "conv_compute" set to 1 or 2 and unit strides the weight gradient is formed
 * from whole zero-padded planes: a non-finite value of x then also meets zeros of dy that belong
 * to a neighbouring channel's or image's positions, and 0 x inf = NaN ends up in the gradient of
 * that neighbouring channel's weights.  Mode 0 confines a non-finite x to its own channel.) */
void conv2d_backward_weight_ecf81c91(const int device_id, const int n, const float* dy, const float* x,
                                     const int accumulate, const int batch, const int channels,
                                     const int height, const int width, const int filters,
                                     const int kernel_h, const int kernel_w, const int pad_h,
                                     const int pad_w, const int stride_h, const int stride_w,
                                     const int dilation_h, const int dilation_w, float* dw);
/* db[filters] (+)= sum of dy over images and pixels; n = filters. */
void conv2d_backward_bias_cd239a08(const int device_id, const int n, const float* dy,
                                   const int accumulate, const int batch, const int pixels, float* db);

/* ---- Library control ---------------------------------------------------- */

/* Per-thread launch stream (a hipStream_t) for subsequent calls; synchronous
 * != 0 makes each call wait for its result before returning. */
void mobula_hip_set_stream(void* stream, int synchronous);

/* Element counts of the NEXT call's arguments, in argument order without the
 * device id, -1 for scalars.  Used to derive N and to reject calls whose
 * buffers cannot hold the problem the scalars describe. */
void mobula_hip_set_arg_extents(const long long* numel, int n);

/* Message of the calling thread's last failed call, or NULL; cleared by
 * mobula_hip_clear_error(). */
const char* mobula_hip_last_error(void);
void mobula_hip_clear_error(void);

/* Named integer switches ("roialign_impl": 0 auto, 1 tiled, 2 naive;
 * "host_staging_device"; "kernel_timing": 0 off, 1 on; "side_stream": 1 (default)
 * lets helper kernels of a call run on a second stream of the device, 0 keeps
 * everything on the caller's stream; "conv_compute": 0 (default) multiplies the
 * convolution's fp32 operands as they are, 1 rounds them to bf16 and accumulates
 * in fp32 (results about 2e-3 off; a non-finite value in x can make the weight
 * gradient of a neighbouring channel NaN, see conv2d_backward_weight), 2 splits
 * every operand into two bf16 and forms three bf16 products per multiply-add
 * (results about 5e-6 off; non-finite values as in mode 1);
 * "roialign_tile_columns": 0 (default) lets the backward pass choose its tile
 * width from the size of the map, 56 or 28 fixes it; "roialign_row_split": 0
 * (default) lets it choose how many wavefronts share a tile row's work list,
 * 1 or 4 fixes it; "roialign_row_quads": 1 (default) lets it write rows of maps
 * whose width is a multiple of four 16 bytes at a time, 0 element by element --
 * all three for tests, the results do not depend on them beyond the order of
 * fp32 sums).  set returns 0, or -1 for an unknown name; get
 * returns -1 for a name never set. */
int mobula_hip_set_option(const char* name, long long value);
long long mobula_hip_get_option(const char* name);

/* With the option "kernel_timing" set to 1 the library brackets the dominant
 * kernel of every operator call (the gather of the forward pass, the tile
 * owners of the backward pass) with HIP events on the launch stream.  Returns
 * the elapsed milliseconds of the calling thread's last bracket after waiting
 * for it, -1 if there is none; *name (if not NULL) receives the kernel's name. */
double mobula_hip_last_kernel_ms(const char** name);

int mobula_hip_device_count(void);

/* The calls keep one grow-only scratch buffer per calling thread and device for
 * their intermediate tables (no counterpart in the reference, whose kernels use
 * none).  workspace_bytes: its current size for the calling thread on the
 * current device.  release_workspace: gives it back to the device (waits for the
 * work that still uses it) and returns the bytes freed; the next call allocates
 * afresh.  A HIP graph recorded from calls of this thread refers to the buffer
 * by address: a call on a capturing stream pins it, and a pinned buffer is
 * neither released nor replaced by a larger one (such a call fails with an
 * error instead) until unpin_workspace() says the graphs are gone.  Replays are
 * not ordered against the thread's calls on other streams (the caller orders those). */
long long mobula_hip_workspace_bytes(void);
long long mobula_hip_release_workspace(void);
void mobula_hip_unpin_workspace(void);

/* 1 if a kernel may dereference p (device, pinned or managed memory), else 0. */
int mobula_hip_device_can_read(const void* p);

/* Space-separated list of the operator entry points in this build. */
const char* mobula_hip_exports(void);

#ifdef __cplusplus
}
#endif
#endif /* MOBULA_ROIALIGN_H_ */
