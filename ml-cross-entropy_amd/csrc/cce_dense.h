// Internal interface between the pieces of the unfiltered backward.
#pragma once

#include "cce_common.h"

namespace cce {

// dz of one vocabulary chunk (cce_dense_dz.hip); the arguments of cce_backward_dz plus `pad_store`: also store
// the zero gradients of the columns between v and ldz.
int dense_dz_launch(const void* e, const void* c, const void* bias,
                    const float* lse, const float* d_out, int d_out_is_scalar, const float* d_lse,
                    const int32_t* valids, const int64_t* targets,
                    void* dz, int64_t ldz, int dz_is_fp32, int pad_store,
                    int64_t n_rows, int64_t b, int64_t v, int64_t d,
                    int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                    float grad_scale, int64_t shift, int64_t target_offset,
                    float softcap, int dtype, hipStream_t stream);

}  // namespace cce
