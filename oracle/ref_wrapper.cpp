/*
 * TEST INFRASTRUCTURE.  Builds the REAL reference ROIAlign kernels, from the
 * sources where they lie under the reference checkout (nothing is copied),
 * into oracle/_ref/.  REF_ROOT is given on the compiler command line as an
 * include directory, see oracle/Makefile.
 *
 * The exported functions are what the reference's loader would generate for
 * the float instantiations, and for the double instantiation of the forward
 * (mobula/op/templates/kernel_code.cpp:1-5 with the names of
 * mobula/func.py:34-50).  The backward has no double instantiation: the
 * reference's atomic_add takes float (context/cpu_ctx.h:37).
 */
#include "mobula_op.h"
using namespace mobula;

#include "opzoo/ROIAlign/ROIAlign.cpp"

extern "C" {

void roi_align_forward_ab78de3c(const int device_id, const int nthreads,
                                const float* bottom_data, const float spatial_scale,
                                const int channels, const int height, const int width,
                                const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const float* bottom_rois,
                                float* top_data) {
  KERNEL_RUN_BEGIN(device_id);
  KERNEL_RUN((roi_align_forward_kernel<float>))
  (nthreads, bottom_data, spatial_scale, channels, height, width, pooled_height,
   pooled_width, sampling_ratio, bottom_rois, top_data);
  KERNEL_RUN_END();
}

void roi_align_forward_6b9e6c9b(const int device_id, const int nthreads,
                                const double* bottom_data, const double spatial_scale,
                                const int channels, const int height, const int width,
                                const int pooled_height, const int pooled_width,
                                const int sampling_ratio, const double* bottom_rois,
                                double* top_data) {
  KERNEL_RUN_BEGIN(device_id);
  KERNEL_RUN((roi_align_forward_kernel<double>))
  (nthreads, bottom_data, spatial_scale, channels, height, width, pooled_height,
   pooled_width, sampling_ratio, bottom_rois, top_data);
  KERNEL_RUN_END();
}

void roi_align_backward_f318a24e(const int device_id, const int nthreads,
                                 const float* top_diff, const float spatial_scale,
                                 const int channels, const int height, const int width,
                                 const int pooled_height, const int pooled_width,
                                 const int sampling_ratio, float* bottom_diff,
                                 const float* bottom_rois) {
  KERNEL_RUN_BEGIN(device_id);
  KERNEL_RUN((roi_align_backward_kernel<float>))
  (nthreads, top_diff, spatial_scale, channels, height, width, pooled_height,
   pooled_width, sampling_ratio, bottom_diff, bottom_rois);
  KERNEL_RUN_END();
}
}
