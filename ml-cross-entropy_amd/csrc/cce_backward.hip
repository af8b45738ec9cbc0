// cce_backward: recompute logit tiles, form softmax - one-hot, filter, accumulate dE / dC / dBias
// on gfx950.
//
// One workgroup (4 waves, 2 x 2) owns one tile of 128 classes x 128 valid rows.
//   1. shortcut   the forward pass left, per 32 rows x 128 classes, the largest soft-capped logit.
//                 If no row of the tile has its target inside the tile and every row's bound
//                 exp(cell_max - lse_row) is below filter_eps, every |p - onehot| of the tile is
//                 below filter_eps as well: the tile is dropped without recomputing it.
//   2. recompute  logits^T = C_tile . E_tile^T with the same LDS-staged MFMA loop as the forward.
//   3. epilogue   p = exp(s - lse), f = p - onehot; the tile is "filtered" iff all |f| < eps;
//                 dz = (p (g + h) - onehot g) (1 - tanh^2), rounded to the input type and written to
//                 LDS twice: [row][class] and [class][row].
//   4. dE         dE[rows] += dz . C_tile, 64 columns of D at a time: A operand = dz from LDS,
//                 B operand gathered column-wise from the staged C chunk; fp32 accumulators go
//                 to HBM with hardware float atomics (fp32 buffer) or packed 16-bit float
//                 atomics (buffer in the input type).
//   5. dC         dC[classes] += dz^T . E_tile, same code with the roles swapped.
#include "cce_common.h"

namespace cce {

struct BwdParams {
  const uint16_t* e;
  const uint16_t* c;
  const uint16_t* bias;
  const float* lse;
  const float* d_out;
  const float* d_lse;
  const int32_t* valids;
  const int32_t* vocab_order;
  const int64_t* targets;
  const float* tile_max;
  void* d_e;
  void* d_c;
  float* d_bias;
  unsigned long long* counters;
  int64_t n_rows, b, v, d;
  int64_t stride_e, stride_cv, stride_cd;
  int64_t shift, target_offset;
  float grad_scale, filter_eps, log_eps;
  int filter_e, filter_c, d_out_is_scalar, de_fp32, dc_fp32;
  int pair_e, pair_c;     // packed two-element 16-bit atomics are legal for dE / dC
  int shortcut;           // tile_max may be used to drop tiles before the recompute
  int nrb, nvt, nitems, items_per_xcd, stat_cols;
  Softcap sc;
};

constexpr int kBwdTile = 128;
constexpr int kGroupRows = 8;  // row blocks per scheduling group

// LDS map (bytes)
constexpr int kOffStage = 0;                       // 64 KB: main-loop stages, later D-chunk buffers
constexpr int kOffDzA = 64 * 1024;                 // 32 KB: dz[row][class]
constexpr int kOffDzB = 96 * 1024;                 // 32 KB: dz[class][row]
constexpr int kOffMeta = 128 * 1024;               // per-row / per-class metadata
constexpr int kBwdLdsBytes = kOffMeta + 6 * 512 + 64;
constexpr int kDzRowBytes = 256;

__device__ __forceinline__ int dz_addr(int row, int col) {
  // 16-byte chunks of a 256-byte row, XOR-swizzled with (row & 7)
  return row * kDzRowBytes + ((((col >> 3) ^ (row & 7)) << 4) | ((col & 7) << 1));
}

// dst[rows given by s_dst] += dz (128 x 128, in LDS) . src[rows given by s_src] over all D columns.
template <typename T, bool ALIGNED>
__device__ __forceinline__ void accumulate_product(const unsigned char* dz, const int* s_src, const uint16_t* src,
                                                   int64_t src_stride_row, int64_t src_stride_col,
                                                   const int* s_dst, void* dst, int64_t dst_stride_row,
                                                   int64_t dst_stride_col, bool dst_fp32, bool pair_ok, int D,
                                                   unsigned char* chunk_lds) {
  using Loader = RowLoader<kBwdTile, 256, ALIGNED>;
  constexpr int kChunkBytes = kBwdTile * kRowBytes;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int half = lane >> 5;

  Loader ld;
#pragma unroll
  for (int q = 0; q < Loader::NQ; ++q) {
    const int id = s_src[(tid >> 3) + q * Loader::ROWSTEP];
    ld.ptr[q] = (id >= 0) ? src + static_cast<int64_t>(id) * src_stride_row : nullptr;
  }
  int dst_id[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) dst_id[r] = s_dst[wave * 32 + 8 * (r >> 2) + 4 * half + (r & 3)];

  const int nchunks = (D + kBK - 1) / kBK;
  ld.load(0, D, src_stride_col);
  ld.store(chunk_lds);
  __syncthreads();

  for (int ci = 0; ci < nchunks; ++ci) {
    const unsigned char* cur = chunk_lds + (ci & 1) * kChunkBytes;
    unsigned char* nxt = chunk_lds + ((ci + 1) & 1) * kChunkBytes;
    const bool more = (ci + 1) < nchunks;
    if (more) ld.load((ci + 1) * kBK, D, src_stride_col);

    f32x16 acc[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[nb][r] = 0.0f;

#pragma unroll
    for (int kk = 0; kk < kBwdTile / 16; ++kk) {
      const int arow = wave * 32 + l32;
      const uint4 araw = *reinterpret_cast<const uint4*>(dz + arow * kDzRowBytes + (((kk * 2 + half) ^ (arow & 7)) << 4));
      const typename Elem<T>::vec8 a = __builtin_bit_cast(typename Elem<T>::vec8, araw);
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        // B operand: 8 consecutive source rows (the reduction index) of one column
        const int col = nb * 32 + l32;
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
          const int r0 = kk * 16 + half * 8 + i;
          const uint16_t lo = *reinterpret_cast<const uint16_t*>(
              cur + r0 * kRowBytes + ((((col >> 3) ^ (r0 & 7)) << 4) | ((col & 7) << 1)));
          const uint16_t hi = *reinterpret_cast<const uint16_t*>(
              cur + (r0 + 1) * kRowBytes + ((((col >> 3) ^ ((r0 + 1) & 7)) << 4) | ((col & 7) << 1)));
          w[i >> 1] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
        }
        const typename Elem<T>::vec8 bfrag = __builtin_bit_cast(typename Elem<T>::vec8, make_uint4(w[0], w[1], w[2], w[3]));
        acc[nb] = Elem<T>::mfma(a, bfrag, acc[nb]);
      }
    }

    // scatter-add the 32 x 64 block of this wave
    const int d0 = ci * kBK;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int col = d0 + nb * 32 + l32;
      if (dst_fp32) {
        float* base = static_cast<float*>(dst);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (dst_id[r] >= 0 && col < D)
            unsafeAtomicAdd(base + static_cast<int64_t>(dst_id[r]) * dst_stride_row + col * dst_stride_col, acc[nb][r]);
        }
      } else if (pair_ok) {
        uint16_t* base = static_cast<uint16_t*>(dst);
        const bool odd = (l32 & 1) != 0;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          // even lane keeps row r, odd lane keeps row r + 1; each gets its neighbour's column
          const float send = odd ? acc[nb][r] : acc[nb][r + 1];
          const float recv = __shfl_xor(send, 1, 64);
          const int id = odd ? dst_id[r + 1] : dst_id[r];
          const float lo = odd ? recv : acc[nb][r];
          const float hi = odd ? acc[nb][r + 1] : recv;
          const int c0 = col & ~1;
          if (id >= 0 && c0 < D) Elem<T>::atomic_add_pair(base + static_cast<int64_t>(id) * dst_stride_row + c0, lo, hi);
        }
      } else {
        uint16_t* base = static_cast<uint16_t*>(dst);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (dst_id[r] >= 0 && col < D)
            atomic_add_16<T>(base + static_cast<int64_t>(dst_id[r]) * dst_stride_row + col * dst_stride_col, acc[nb][r]);
        }
      }
    }

    if (more) ld.store(nxt);
    __syncthreads();
  }
}

template <typename T, bool ALIGNED>
__global__ __launch_bounds__(256, 1) void backward_kernel(BwdParams p) {
  using Tile = LogitTile<T, 2, 2, 2, 2, ALIGNED>;
  extern __shared__ __align__(16) unsigned char smem[];
  int* s_row = reinterpret_cast<int*>(smem + kOffMeta);          // E row of each tile row, -1: none
  int* s_cid = s_row + 128;                                      // class id of each tile column, -1: none
  int* s_tgt = s_cid + 128;                                      // target class of each tile row, -2: none
  float* s_lse2 = reinterpret_cast<float*>(s_tgt + 128);         // lse * log2(e), +inf: none
  float* s_g = s_lse2 + 128;                                     // grad_scale * d_out
  float* s_h = s_g + 128;                                        // d_lse

  // XCD-aware tile id, then grouped ordering: kGroupRows row blocks sweep the vocabulary together.
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  if (slot >= p.items_per_xcd) return;
  const int item = xcd * p.items_per_xcd + slot;
  if (item >= p.nitems) return;
  const int per_group = kGroupRows * p.nvt;
  const int group = item / per_group;
  const int first_rb = group * kGroupRows;
  const int gsize = min(p.nrb - first_rb, kGroupRows);
  const int rb = first_rb + (item % per_group) % gsize;
  const int vt = (item % per_group) / gsize;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wv = wave >> 1;
  const int wt = wave & 1;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int64_t t0 = static_cast<int64_t>(rb) * kBwdTile;
  const int64_t v0 = static_cast<int64_t>(vt) * kBwdTile;

  if (item == 0 && tid == 0 && p.counters != nullptr)
    atomicAdd(p.counters + 0, static_cast<unsigned long long>(p.nitems));

  // ---- metadata ----------------------------------------------------------------------------
  bool keep = false;
  if (tid < 128) {
    const int64_t i = t0 + tid;
    int row = -1, tgt = -2;
    float lse2 = INFINITY, g = 0.0f, h = 0.0f;
    if (i < p.b) {
      const int64_t rr = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
      row = static_cast<int>(rr);
      const float lse = p.lse[i];
      lse2 = lse * kLog2e;
      const int64_t ti = rr + p.shift;
      if (ti < p.n_rows) {
        const int64_t t = p.targets[ti] - p.target_offset;
        if (t >= 0 && t < p.v) tgt = static_cast<int>(t);
        g = p.grad_scale * (p.d_out_is_scalar ? p.d_out[0] : p.d_out[ti]);
        if (p.d_lse != nullptr) h = p.d_lse[ti];
      }
      if (p.shortcut) {
        const bool hit = (tgt >= v0) && (tgt < v0 + kBwdTile);
        const float cell = p.tile_max[((t0 + tid) / CCE_STAT_ROWS) * p.stat_cols + v0 / CCE_STAT_COLS];
        keep = hit || (cell - lse >= p.log_eps);
      }
    }
    s_row[tid] = row;
    s_tgt[tid] = tgt;
    s_lse2[tid] = lse2;
    s_g[tid] = g;
    s_h[tid] = h;
  } else {
    const int64_t pos = v0 + (tid - 128);
    int cid = -1;
    if (pos < p.v) cid = p.vocab_order ? p.vocab_order[pos] : static_cast<int>(pos);
    s_cid[tid - 128] = cid;
  }
  if (p.shortcut) {
    if (!__syncthreads_or(keep ? 1 : 0)) return;
  } else {
    __syncthreads();
  }
  if (tid == 0 && p.counters != nullptr) atomicAdd(p.counters + 1, 1ull);

  // ---- recompute the logit tile ----------------------------------------------------------------
  typename Tile::CLoader cl;
  typename Tile::ELoader el;
#pragma unroll
  for (int q = 0; q < Tile::CLoader::NQ; ++q) {
    const int cid = s_cid[(tid >> 3) + q * Tile::CLoader::ROWSTEP];
    cl.ptr[q] = (cid >= 0) ? p.c + static_cast<int64_t>(cid) * p.stride_cv : nullptr;
    const int row = s_row[(tid >> 3) + q * Tile::ELoader::ROWSTEP];
    el.ptr[q] = (row >= 0) ? p.e + static_cast<int64_t>(row) * p.stride_e : nullptr;
  }
  f32x16 acc[2][2];
  Tile::run(acc, cl, el, smem + kOffStage, static_cast<int>(p.d), p.stride_cd);

  // ---- epilogue ------------------------------------------------------------------------------
  float lse2[2], g[2], h[2];
  int tgt[2];
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    const int tj = wt * 64 + ti * 32 + l32;
    lse2[ti] = s_lse2[tj];
    g[ti] = s_g[tj];
    h[ti] = s_h[tj];
    tgt[ti] = s_tgt[tj];
  }
  const float eps = p.filter_eps;
  bool big = false;
#pragma unroll
  for (int vi = 0; vi < 2; ++vi) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int lv = wv * 64 + vi * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
      const int cid = s_cid[lv];
      float bias = 0.0f;
      if (p.bias != nullptr && cid >= 0) bias = Elem<T>::to_float(p.bias[cid]);
#pragma unroll
      for (int ti = 0; ti < 2; ++ti) {
        float th;
        const float s2 = softcap_log2(p.sc, acc[vi][ti][r] + bias, th);
        const float pr = (cid >= 0) ? __builtin_amdgcn_exp2f(s2 - lse2[ti]) : 0.0f;
        const bool hit = (cid >= 0) && (cid == tgt[ti]);
        const float f = pr - (hit ? 1.0f : 0.0f);
        big = big || (fabsf(f) >= eps);
        float dz = pr * (g[ti] + h[ti]) - (hit ? g[ti] : 0.0f);
        if (p.sc.on) dz *= (1.0f - th * th);
        acc[vi][ti][r] = dz;
      }
    }
  }
  bool filtered = false;
  if (eps >= 0.0f) filtered = (__syncthreads_or(big ? 1 : 0) == 0);
  const bool do_e = (p.d_e != nullptr) && !(p.filter_e && filtered);
  const bool do_c = (p.d_c != nullptr) && !(p.filter_c && filtered);
  const bool do_b = (p.d_bias != nullptr) && !(p.filter_e && p.filter_c && filtered);
  if (!do_e && !do_c && !do_b) return;
  if (tid == 0 && p.counters != nullptr) {
    if (do_e) atomicAdd(p.counters + 2, 1ull);
    if (do_c) atomicAdd(p.counters + 3, 1ull);
  }

  if (do_b) {
#pragma unroll
    for (int vi = 0; vi < 2; ++vi) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int lv = wv * 64 + vi * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
        float colsum = acc[vi][0][r] + acc[vi][1][r];
#pragma unroll
        for (int off = 16; off >= 1; off >>= 1) colsum += __shfl_xor(colsum, off, 64);
        const int cid = s_cid[lv];
        if (l32 == 0 && cid >= 0) unsafeAtomicAdd(p.d_bias + cid, colsum);
      }
    }
  }

  if (do_e || do_c) {
    unsigned char* dzA = smem + kOffDzA;  // [row][class]
    unsigned char* dzB = smem + kOffDzB;  // [class][row]
#pragma unroll
    for (int vi = 0; vi < 2; ++vi) {
#pragma unroll
      for (int ti = 0; ti < 2; ++ti) {
        const int tj = wt * 64 + ti * 32 + l32;
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int lv = wv * 64 + vi * 32 + 8 * r4 + 4 * half;
          uint16_t q[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            q[i] = Elem<T>::from_float(acc[vi][ti][r4 * 4 + i]);
            *reinterpret_cast<uint16_t*>(dzB + dz_addr(lv + i, tj)) = q[i];
          }
          uint2 packed;
          packed.x = static_cast<uint32_t>(q[0]) | (static_cast<uint32_t>(q[1]) << 16);
          packed.y = static_cast<uint32_t>(q[2]) | (static_cast<uint32_t>(q[3]) << 16);
          *reinterpret_cast<uint2*>(dzA + dz_addr(tj, lv)) = packed;
        }
      }
    }
    __syncthreads();

    if (do_e) {
      accumulate_product<T, ALIGNED>(dzA, s_cid, p.c, p.stride_cv, p.stride_cd, s_row, p.d_e, p.stride_e, 1,
                                     p.de_fp32 != 0, p.pair_e != 0, static_cast<int>(p.d), smem + kOffStage);
    }
    if (do_c) {
      accumulate_product<T, ALIGNED>(dzB, s_row, p.e, p.stride_e, 1, s_cid, p.d_c, p.stride_cv, p.stride_cd,
                                     p.dc_fp32 != 0, p.pair_c != 0, static_cast<int>(p.d), smem + kOffStage);
    }
  }
}

}  // namespace cce

using namespace cce;

extern "C" int64_t cce_backward_workspace_bytes(int64_t b, int64_t v, int64_t d) {
  (void)b;
  (void)v;
  (void)d;
  return 0;
}

extern "C" int cce_backward(const void* e, const void* c, const void* bias,
                            const float* lse, const float* d_out, int d_out_is_scalar, const float* d_lse,
                            const int32_t* valids, const int32_t* vocab_order, const int64_t* targets,
                            const float* tile_max,
                            void* d_e, void* d_c, float* d_bias,
                            void* workspace, int64_t workspace_bytes, uint64_t* counters,
                            int64_t n_rows, int64_t b, int64_t v, int64_t d,
                            int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                            float grad_scale, float filter_eps, int filter_e, int filter_c,
                            int d_e_is_fp32, int d_c_is_fp32,
                            int64_t shift, int64_t target_offset,
                            float softcap, int dtype, void* stream_) {
  (void)workspace;
  (void)workspace_bytes;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (b < 0 || v <= 0 || d <= 0 || n_rows < 0 || shift < 0) return CCE_ERR_INVALID_ARGUMENT;
  if (b == 0) return CCE_OK;
  if (e == nullptr || c == nullptr || lse == nullptr || d_out == nullptr || targets == nullptr)
    return CCE_ERR_INVALID_ARGUMENT;
  if (valids == nullptr && b > n_rows) return CCE_ERR_INVALID_ARGUMENT;
  if (n_rows >= (int64_t(1) << 31) || v >= (int64_t(1) << 31) - 512 || d > (1 << 30)) return CCE_ERR_INVALID_ARGUMENT;
  if (dtype != CCE_DTYPE_BF16 && dtype != CCE_DTYPE_F16) return CCE_ERR_UNSUPPORTED_DTYPE;
  if (d_e == nullptr && d_c == nullptr && d_bias == nullptr) return CCE_OK;

  BwdParams p;
  p.e = static_cast<const uint16_t*>(e);
  p.c = static_cast<const uint16_t*>(c);
  p.bias = static_cast<const uint16_t*>(bias);
  p.lse = lse;
  p.d_out = d_out;
  p.d_lse = d_lse;
  p.valids = valids;
  p.vocab_order = vocab_order;
  p.targets = targets;
  p.tile_max = tile_max;
  p.d_e = d_e;
  p.d_c = d_c;
  p.d_bias = d_bias;
  p.counters = reinterpret_cast<unsigned long long*>(counters);
  p.n_rows = n_rows;
  p.b = b;
  p.v = v;
  p.d = d;
  p.stride_e = stride_e;
  p.stride_cv = stride_cv;
  p.stride_cd = stride_cd;
  p.shift = shift;
  p.target_offset = target_offset;
  p.grad_scale = grad_scale;
  const bool filtering = filter_eps >= 0.0f;
  p.filter_eps = filtering ? filter_eps : -1.0f;
  p.filter_e = (filtering && filter_e) ? 1 : 0;
  p.filter_c = (filtering && filter_c) ? 1 : 0;
  // a bound just under eps keeps the tile: a little slack costs a recompute, never an error
  p.log_eps = (filtering && filter_eps > 0.0f) ? logf(filter_eps) - 0.01f : -INFINITY;
  p.d_out_is_scalar = d_out_is_scalar;
  p.de_fp32 = d_e_is_fp32;
  p.dc_fp32 = d_c_is_fp32;
  p.pair_e = (!d_e_is_fp32 && d_e != nullptr && (d % 2 == 0) && (stride_e % 2 == 0) &&
              (reinterpret_cast<uintptr_t>(d_e) % 4 == 0)) ? 1 : 0;
  p.pair_c = (!d_c_is_fp32 && d_c != nullptr && (d % 2 == 0) && (stride_cv % 2 == 0) && stride_cd == 1 &&
              (reinterpret_cast<uintptr_t>(d_c) % 4 == 0)) ? 1 : 0;
  // The shortcut is sound only when a filtered tile contributes to nothing that was asked for.
  const bool all_filtered = (d_e == nullptr || p.filter_e) && (d_c == nullptr || p.filter_c) &&
                            (d_bias == nullptr || (p.filter_e && p.filter_c));
  p.shortcut = (tile_max != nullptr && vocab_order == nullptr && filtering && filter_eps > 0.0f && all_filtered) ? 1 : 0;
  p.nrb = static_cast<int>((b + kBwdTile - 1) / kBwdTile);
  p.nvt = static_cast<int>((v + kBwdTile - 1) / kBwdTile);
  const int64_t nitems = static_cast<int64_t>(p.nrb) * p.nvt;
  if (nitems > (int64_t(1) << 30)) return CCE_ERR_INVALID_ARGUMENT;
  p.nitems = static_cast<int>(nitems);
  p.items_per_xcd = (p.nitems + 7) / 8;
  p.stat_cols = static_cast<int>((v + CCE_STAT_COLS - 1) / CCE_STAT_COLS);
  p.sc = make_softcap(softcap);

  const bool aligned = aligned16(e) && aligned16(c) && (d % 8 == 0) && (stride_e % 8 == 0) &&
                       (stride_cv % 8 == 0) && (stride_cd == 1);
  const dim3 grid(static_cast<unsigned>(p.items_per_xcd) * 8u);
  hipError_t err;
#define CCE_LAUNCH_BWD(TT, AL)                                                                     \
  do {                                                                                             \
    auto kern = backward_kernel<TT, AL>;                                                           \
    err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                 \
                              hipFuncAttributeMaxDynamicSharedMemorySize, kBwdLdsBytes);           \
    if (err != hipSuccess) return status_from_hip(err);                                            \
    hipLaunchKernelGGL(kern, grid, dim3(256), kBwdLdsBytes, stream, p);                            \
  } while (0)
  if (dtype == CCE_DTYPE_BF16) {
    if (aligned) CCE_LAUNCH_BWD(BF16, true); else CCE_LAUNCH_BWD(BF16, false);
  } else {
    if (aligned) CCE_LAUNCH_BWD(F16, true); else CCE_LAUNCH_BWD(F16, false);
  }
#undef CCE_LAUNCH_BWD
  return status_from_hip(hipGetLastError());
}
