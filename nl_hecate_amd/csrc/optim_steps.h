// Pieces of the optimizer step shared by optim.hip (the kernels) and cms.hip (the frequency-aware driver).
#pragma once

namespace nlh {

// norm of a set of gradient tensors and the clip factor min(1, max_grad_norm / norm), both left on the device
unsigned grad_norm_scale_multi(float *const *g, const int *n, int count, float max_grad_norm, float *out_norm,
                               float *out_scale);
// every tensor times *scale_ptr in place when that is below 1
unsigned grad_scale_multi(float *const *g, const int *n, int count, const float *scale_ptr);
// adamw_update_multi_rocm with the gradients first multiplied by *scale_ptr (when below 1; null: no scaling) and
// written back: one pass over the gradients instead of a scaling pass and an update pass
unsigned adamw_update_multi_scaled(float *const *w, const float *const *g, float *const *m, float *const *v,
                                   const int *n, const float *bc1_inv, const float *bc2_inv, int count, float lr,
                                   float beta1, float beta2, float eps, float weight_decay, const float *scale_ptr);

}  // namespace nlh
