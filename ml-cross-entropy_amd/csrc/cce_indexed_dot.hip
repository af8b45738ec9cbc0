// cce_indexed_neg_dot: out[i] = softcap(-(E[row_i] . C[t_i]) - bias[t_i]) for gfx950.
//
// HBM-bound gather-dot: one wavefront per valid row streams the row of E and the row of C its
// target selects with 16-byte loads (lane l reads elements 8 l .. 8 l + 7 of every 512-element
// stripe, so a wave reads whole contiguous kilobytes), multiplies in fp32 and reduces across the
// wave with shuffles.  The bias is subtracted exactly once per row and soft-capping is fused.
#include "cce_common.h"

namespace cce {

struct IdxDotParams {
  const uint16_t* e;
  const uint16_t* c;
  const int64_t* targets;
  const uint16_t* bias;
  const int32_t* valids;
  float* out;
  int64_t n_rows, b, v, d;
  int64_t stride_e, stride_cv, stride_cd;
  int64_t shift, target_offset;
  float softcap;
};

template <typename T, bool ALIGNED>
__global__ __launch_bounds__(256) void indexed_neg_dot_kernel(IdxDotParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (i >= p.b) return;
  const int64_t row = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
  const int64_t ti = row + p.shift;
  int64_t t = -1;
  if (ti >= 0 && ti < p.n_rows) t = p.targets[ti] - p.target_offset;
  if (t < 0 || t >= p.v) {  // wave-uniform: masked rows contribute an exact zero
    if (lane == 0) p.out[i] = 0.0f;
    return;
  }
  const uint16_t* er = p.e + row * p.stride_e;
  const uint16_t* cr = p.c + t * p.stride_cv;
  float acc = 0.0f;
  if (ALIGNED) {
    for (int64_t k = lane * 8; k < p.d; k += 512) {
      const uint4 a = *reinterpret_cast<const uint4*>(er + k);
      const uint4 b = *reinterpret_cast<const uint4*>(cr + k);
      const uint32_t aw[4] = {a.x, a.y, a.z, a.w};
      const uint32_t bw[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc += Elem<T>::to_float(static_cast<uint16_t>(aw[j] & 0xffffu)) *
               Elem<T>::to_float(static_cast<uint16_t>(bw[j] & 0xffffu));
        acc += Elem<T>::to_float(static_cast<uint16_t>(aw[j] >> 16)) *
               Elem<T>::to_float(static_cast<uint16_t>(bw[j] >> 16));
      }
    }
  } else {
    for (int64_t k = lane; k < p.d; k += 64)
      acc += Elem<T>::to_float(er[k]) * Elem<T>::to_float(cr[k * p.stride_cd]);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) {
    float r = -acc;
    if (p.bias != nullptr) r -= Elem<T>::to_float(p.bias[t]);
    if (p.softcap > 0.0f) r = tanhf(r / p.softcap) * p.softcap;
    p.out[i] = r;
  }
}

}  // namespace cce

using namespace cce;

extern "C" int cce_indexed_neg_dot(const void* e, const void* c, const int64_t* targets, const void* bias,
                                   const int32_t* valids, float* out,
                                   int64_t n_rows, int64_t b, int64_t v, int64_t d,
                                   int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                                   int64_t shift, int64_t target_offset,
                                   float softcap, int dtype, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (b < 0 || v <= 0 || d <= 0 || n_rows < 0 || shift < 0) return CCE_ERR_INVALID_ARGUMENT;
  if (b == 0) return CCE_OK;
  if (e == nullptr || c == nullptr || targets == nullptr || out == nullptr) return CCE_ERR_INVALID_ARGUMENT;
  if (valids == nullptr && b > n_rows) return CCE_ERR_INVALID_ARGUMENT;
  if (dtype != CCE_DTYPE_BF16 && dtype != CCE_DTYPE_F16) return CCE_ERR_UNSUPPORTED_DTYPE;

  IdxDotParams p;
  p.e = static_cast<const uint16_t*>(e);
  p.c = static_cast<const uint16_t*>(c);
  p.targets = targets;
  p.bias = static_cast<const uint16_t*>(bias);
  p.valids = valids;
  p.out = out;
  p.n_rows = n_rows;
  p.b = b;
  p.v = v;
  p.d = d;
  p.stride_e = stride_e;
  p.stride_cv = stride_cv;
  p.stride_cd = stride_cd;
  p.shift = shift;
  p.target_offset = target_offset;
  p.softcap = softcap;

  const bool aligned = aligned16(e) && aligned16(c) && (d % 8 == 0) && (stride_e % 8 == 0) &&
                       (stride_cv % 8 == 0) && (stride_cd == 1);
  const dim3 grid(static_cast<unsigned>((b + 3) / 4));
  if (dtype == CCE_DTYPE_BF16) {
    if (aligned) hipLaunchKernelGGL((indexed_neg_dot_kernel<BF16, true>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((indexed_neg_dot_kernel<BF16, false>), grid, dim3(256), 0, stream, p);
  } else {
    if (aligned) hipLaunchKernelGGL((indexed_neg_dot_kernel<F16, true>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((indexed_neg_dot_kernel<F16, false>), grid, dim3(256), 0, stream, p);
  }
  return status_from_hip(hipGetLastError());
}
