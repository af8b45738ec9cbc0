// cce_backward: recompute logit tiles, form softmax - one-hot, filter, accumulate dE / dC / dBias
// on gfx950 -- without a single global atomic on the gradients.
//
// Global read-modify-write is the slow path of this chip (a few hundred G lane-updates/s), so the
// two gradients are produced by two ownership kernels whose accumulators never leave registers:
//
//   bwd_de_kernel   one workgroup (4 waves) owns 32 valid rows (a "row group") and up to 2304
//                   columns of dE.  It walks the 128-class cells of the vocabulary that can matter
//                   for its rows, recomputes logits^T (128 classes x 32 rows) with MFMA, forms
//                   dz, applies the gradient filter per 32 x 32 sub-tile, and accumulates
//                   dE^T (D x 32 rows) += C_cell^T . dz^T in fp32 registers (wave w owns the 32-column
//                   blocks w, w + 4 of every 256).  The rows are written once at the end.  It also records,
//                   one bit per 32 x 32 sub-tile, which sub-tiles survived the filter.
//   bwd_dc_kernel   one workgroup owns 32 classes (and up to 2304 columns of dC), walks the row
//                   groups whose bit is set (all of them when dC is not filtered), recomputes the
//                   32 x 32 logits, and accumulates dC^T (D x 32 classes) += E_group^T . dz; dBias is
//                   the row sum of the same dz.  Rows are written once at the end.
//
// Which cells can matter: the forward pass left, per 32 rows x 128 classes, the largest soft-capped
// logit.  A cell none of whose rows has its target inside and whose bound
// exp(cell_max - min_row lse) is below filter_eps has every |p - onehot| below filter_eps, so the
// filter would drop all four of its sub-tiles: it is skipped without being recomputed.
//
// The price of ownership is that kept sub-tiles are recomputed once more in the second kernel;
// with filtering that is a small fraction of the plane.  Results are deterministic.
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
  uint32_t* kept_bits;  // [ntg][bit_words]: bit (vg % 32) of word vg / 32 <=> sub-tile (tg, vg) survived
  unsigned long long* counters;
  int64_t n_rows, b, v, d;
  int64_t stride_e, stride_cv, stride_cd;
  int64_t shift, target_offset;
  float grad_scale, filter_eps, log_eps;
  int filter_e, filter_c, d_out_is_scalar, de_fp32, dc_fp32;
  int shortcut;  // tile_max may be used to skip cells before the recompute
  int ntg, nvc, nvg, bit_words, nslices, dslice, stat_cols;
  int vec_e, vec_c;  // 4-element vector stores are legal for dE / dC
  Softcap sc;
};

constexpr int kStageCols = 256;               // columns of D per LDS stage
constexpr int kStageRowBytes = kStageCols * 2;
constexpr int kMaxChunks = 9;                 // 9 * 256 = 2304 columns of D per workgroup
constexpr int kListCap = 4096;                // cells / row groups listed per pass
constexpr int kBwdThreads = 256;              // 4 waves, one per SIMD: each may use all 512 registers

__device__ __forceinline__ int stage_addr(int row, int col) {
  return row * kStageRowBytes + ((((col >> 3) ^ (row & 7)) << 4) | ((col & 7) << 1));
}

// R rows x 256 columns, global -> registers -> LDS.  Thread t owns 16-byte chunk (t & 31) of rows
// (t >> 5) + 8 q.  Rows come from an id table in LDS (id < 0: no row); a 32-row block whose bit in
// `block_mask` is clear is neither loaded nor stored.
template <int R, bool ALIGNED>
struct StageLoader {
  static constexpr int NQ = R / 8;
  uint4 reg[NQ];

  __device__ __forceinline__ void load(const int* ids, const uint16_t* base, int64_t stride_row, int64_t stride_col,
                                       int col0, int D, uint32_t block_mask) {
    const int k = col0 + (threadIdx.x & 31) * 8;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int row = (threadIdx.x >> 5) + 8 * q;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      const int id = ids[row];
      if (id >= 0 && ((block_mask >> (row >> 5)) & 1u)) {
        const uint16_t* ptr = base + static_cast<int64_t>(id) * stride_row;
        if (ALIGNED) {
          if (k < D) v = *reinterpret_cast<const uint4*>(ptr + k);
        } else {
          uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const uint32_t x = (k + i < D) ? static_cast<uint32_t>(ptr[static_cast<int64_t>(k + i) * stride_col]) : 0u;
            w[i >> 1] |= x << ((i & 1) * 16);
          }
          v = make_uint4(w[0], w[1], w[2], w[3]);
        }
      }
      reg[q] = v;
    }
  }

  __device__ __forceinline__ void store(unsigned char* lds, uint32_t block_mask) const {
    const int chunk = threadIdx.x & 31;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int row = (threadIdx.x >> 5) + 8 * q;
      if ((block_mask >> (row >> 5)) & 1u)
        *reinterpret_cast<uint4*>(lds + row * kStageRowBytes + ((chunk ^ (row & 7)) << 4)) = reg[q];
    }
  }
};

template <typename T>
__device__ __forceinline__ typename Elem<T>::vec8 stage_frag(const unsigned char* lds, int row, int chunk) {
  const uint4 v = *reinterpret_cast<const uint4*>(lds + row * kStageRowBytes + ((chunk ^ (row & 7)) << 4));
  return __builtin_bit_cast(typename Elem<T>::vec8, v);
}

// MFMA operand whose reduction index runs over 8 consecutive stage rows r0 .. r0 + 7 of column `col`.
template <typename T>
__device__ __forceinline__ typename Elem<T>::vec8 stage_frag_transposed(const unsigned char* lds, int r0, int col) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    const uint32_t lo = *reinterpret_cast<const uint16_t*>(lds + stage_addr(r0 + i, col));
    const uint32_t hi = *reinterpret_cast<const uint16_t*>(lds + stage_addr(r0 + i + 1, col));
    w[i >> 1] = lo | (hi << 16);
  }
  return __builtin_bit_cast(typename Elem<T>::vec8, make_uint4(w[0], w[1], w[2], w[3]));
}

// Write the fp32 accumulators of one wave (lane = destination row, registers = 32 columns starting
// at col0) to a gradient matrix, converting to the buffer type.
template <typename T>
__device__ __forceinline__ void store_rows(const f32x16& acc, void* dst, bool fp32, bool vec_ok, int64_t row_off,
                                           int64_t stride_col, int col0, int half, int D) {
#pragma unroll
  for (int r4 = 0; r4 < 4; ++r4) {
    const int col = col0 + 8 * r4 + 4 * half;
    if (fp32) {
      float* base = static_cast<float*>(dst) + row_off;
      if (vec_ok && col + 3 < D) {
        *reinterpret_cast<float4*>(base + col) =
            make_float4(acc[r4 * 4 + 0], acc[r4 * 4 + 1], acc[r4 * 4 + 2], acc[r4 * 4 + 3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col + i < D) base[static_cast<int64_t>(col + i) * stride_col] = acc[r4 * 4 + i];
      }
    } else {
      uint16_t* base = static_cast<uint16_t*>(dst) + row_off;
      uint16_t q[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) q[i] = Elem<T>::from_float(acc[r4 * 4 + i]);
      if (vec_ok && col + 3 < D) {
        uint2 pk;
        pk.x = static_cast<uint32_t>(q[0]) | (static_cast<uint32_t>(q[1]) << 16);
        pk.y = static_cast<uint32_t>(q[2]) | (static_cast<uint32_t>(q[3]) << 16);
        *reinterpret_cast<uint2*>(base + col) = pk;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (col + i < D) base[static_cast<int64_t>(col + i) * stride_col] = q[i];
      }
    }
  }
}

// Per-row metadata of one row group, written by threads 0..31.
struct RowMeta {
  int* row;      // row of E, -1: none
  int* tgt;      // target class (after the shard offset), -2: none
  float* lse2;   // lse * log2(e), +inf: none
  float* g;      // grad_scale * d_out
  float* h;      // d_lse
};

__device__ __forceinline__ float load_row_meta(const BwdParams& p, int64_t i, int slot, const RowMeta& m) {
  int row = -1, tgt = -2;
  float lse2 = INFINITY, g = 0.0f, h = 0.0f, lse = INFINITY;
  if (i < p.b) {
    const int64_t rr = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
    row = static_cast<int>(rr);
    lse = p.lse[i];
    lse2 = lse * kLog2e;
    const int64_t ti = rr + p.shift;
    if (ti < p.n_rows) {
      const int64_t t = p.targets[ti] - p.target_offset;
      if (t >= 0 && t < p.v) tgt = static_cast<int>(t);
      g = p.grad_scale * (p.d_out_is_scalar ? p.d_out[0] : p.d_out[ti]);
      if (p.d_lse != nullptr) h = p.d_lse[ti];
    }
  }
  m.row[slot] = row;
  m.tgt[slot] = tgt;
  m.lse2[slot] = lse2;
  m.g[slot] = g;
  m.h[slot] = h;
  return lse;
}

// One 32 x 32 block of logits^T (lane = row `l32` of the group, registers = classes) -> dz.
// Returns whether any |p - onehot| reaches eps.
template <typename T>
__device__ __forceinline__ bool block_epilogue(const BwdParams& p, f32x16& acc, const int* cid32, int half,
                                               float lse2, float g, float h, int tgt) {
  bool big = false;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int cid = cid32[8 * (r >> 2) + 4 * half + (r & 3)];
    float bias = 0.0f;
    if (p.bias != nullptr && cid >= 0) bias = Elem<T>::to_float(p.bias[cid]);
    float th;
    const float s2 = softcap_log2(p.sc, acc[r] + bias, th);
    const float pr = (cid >= 0) ? __builtin_amdgcn_exp2f(s2 - lse2) : 0.0f;
    const bool hit = (cid >= 0) && (cid == tgt);
    const float f = pr - (hit ? 1.0f : 0.0f);
    big = big || (fabsf(f) >= p.filter_eps);
    float dz = pr * (g + h) - (hit ? g : 0.0f);
    if (p.sc.on) dz *= (1.0f - th * th);
    acc[r] = dz;
  }
  return big;
}

// ---------------------------------------------------------------------------------------------
// dE: workgroup = (row group of 32, slice of D)
// ---------------------------------------------------------------------------------------------
constexpr int kDeOffC = 0;                          // 64 KB  C stage: 128 classes x 256 columns
constexpr int kDeOffE = 64 * 1024;                  // 16 KB  E stage: 32 rows x 256 columns
constexpr int kDeOffDz = 80 * 1024;                 //  8 KB  dz^T [row][class], 256 bytes per row
constexpr int kDeOffList = 88 * 1024;               // 16 KB  cell list
constexpr int kDeOffFlag = 104 * 1024;              //  4 KB  cell flags (bytes)
constexpr int kDeOffBits = 108 * 1024;              //  bit row, then metadata
constexpr int kDeMaxBitWords = 2048;                //  8 KB  (V <= 2 M classes)
constexpr int kDeOffMeta = kDeOffBits + kDeMaxBitWords * 4;
constexpr int kDeLdsBytes = kDeOffMeta + 5 * 128 + 512 + 64;

template <typename T, bool ALIGNED>
__global__ __launch_bounds__(kBwdThreads, 1) void bwd_de_kernel(BwdParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sC = smem + kDeOffC;
  unsigned char* sE = smem + kDeOffE;
  unsigned char* sDz = smem + kDeOffDz;
  int* sList = reinterpret_cast<int*>(smem + kDeOffList);
  unsigned char* sFlag = smem + kDeOffFlag;
  uint32_t* sBits = reinterpret_cast<uint32_t*>(smem + kDeOffBits);
  RowMeta meta;
  meta.row = reinterpret_cast<int*>(smem + kDeOffMeta);
  meta.tgt = meta.row + 32;
  meta.lse2 = reinterpret_cast<float*>(meta.tgt + 32);
  meta.g = meta.lse2 + 32;
  meta.h = meta.g + 32;
  int* sCid = reinterpret_cast<int*>(meta.h + 32);  // [128]
  int* sMisc = sCid + 128;                           // [0] list length, [1] kept-block mask, [2] min lse

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int tg = blockIdx.x / p.nslices;
  const int slice = blockIdx.x % p.nslices;
  const int d_begin = slice * p.dslice;
  const int d_end = min(static_cast<int>(p.d), d_begin + p.dslice);
  const int nchunks = (d_end - d_begin + kStageCols - 1) / kStageCols;
  const int D = static_cast<int>(p.d);
  const bool write_de = (p.d_e != nullptr);

  // ---- row metadata, minimum lse of the group ------------------------------------------------
  float my_lse = INFINITY;
  if (tid < 32) my_lse = load_row_meta(p, static_cast<int64_t>(tg) * 32 + tid, tid, meta);
  if (wave == 0) {
    const float mn = wave_min(my_lse);
    if (lane == 0) reinterpret_cast<float*>(sMisc)[2] = mn;
  }
  for (int w = tid; w < p.bit_words; w += kBwdThreads) sBits[w] = 0u;
  __syncthreads();
  const float min_lse = reinterpret_cast<float*>(sMisc)[2];

  // wave w owns columns [32 w, 32 w + 32) and [128 + 32 w, 128 + 32 w + 32) of every 256-column chunk
  f32x16 acc[kMaxChunks][2];
#pragma unroll
  for (int ci = 0; ci < kMaxChunks; ++ci)
#pragma unroll
    for (int hb = 0; hb < 2; ++hb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ci][hb][r] = 0.0f;

  unsigned long long n_recomputed = 0, n_product = 0;

  for (int seg = 0; seg < p.nvc; seg += kListCap) {
    const int seg_n = min(kListCap, p.nvc - seg);
    // ---- which cells of this segment have to be recomputed ------------------------------------
    if (p.shortcut) {
      for (int j = tid; j < seg_n; j += kBwdThreads) {
        const float cell = p.tile_max[static_cast<int64_t>(tg) * p.stat_cols + seg + j];
        sFlag[j] = (cell - min_lse >= p.log_eps) ? 1 : 0;
      }
      __syncthreads();
      if (tid < 32) {
        const int t = meta.tgt[tid];
        if (t >= 0) {
          const int cell = t / 128 - seg;
          if (cell >= 0 && cell < seg_n) sFlag[cell] = 1;
        }
      }
      __syncthreads();
      if (wave == 0) {  // ordered compaction: the accumulation order, hence the result, is fixed
        int n = 0;
        for (int base = 0; base < seg_n; base += 64) {
          const bool f = (base + lane < seg_n) && (sFlag[base + lane] != 0);
          const unsigned long long m = __ballot(f);
          if (f) sList[n + __popcll(m & ((1ull << lane) - 1ull))] = seg + base + lane;
          n += __popcll(m);
        }
        if (lane == 0) sMisc[0] = n;
      }
      __syncthreads();
    }
    const int list_n = p.shortcut ? sMisc[0] : seg_n;

    for (int li = 0; li < list_n; ++li) {
      const int vc = p.shortcut ? sList[li] : seg + li;
      // ---- class ids of the cell ---------------------------------------------------------------
      if (tid < 128) {
        const int64_t pos = static_cast<int64_t>(vc) * 128 + tid;
        int cid = -1;
        if (pos < p.v) cid = p.vocab_order ? p.vocab_order[pos] : static_cast<int>(pos);
        sCid[tid] = cid;
      }
      if (tid == 0) sMisc[1] = 0;
      __syncthreads();

      // ---- logits^T (128 classes x 32 rows): wave w = classes [32 w, 32 w + 32) -----------------------
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.0f;
      {
        StageLoader<128, ALIGNED> lc;
        StageLoader<32, ALIGNED> le;
        const int nstages = (D + kStageCols - 1) / kStageCols;
        lc.load(sCid, p.c, p.stride_cv, p.stride_cd, 0, D, 0xfu);
        le.load(meta.row, p.e, p.stride_e, 1, 0, D, 0x1u);
        for (int st = 0; st < nstages; ++st) {
          lc.store(sC, 0xfu);
          le.store(sE, 0x1u);
          __syncthreads();
          if (st + 1 < nstages) {
            lc.load(sCid, p.c, p.stride_cv, p.stride_cd, (st + 1) * kStageCols, D, 0xfu);
            le.load(meta.row, p.e, p.stride_e, 1, (st + 1) * kStageCols, D, 0x1u);
          }
#pragma unroll
          for (int kk = 0; kk < 16; ++kk) {
            const auto a = stage_frag<T>(sC, wave * 32 + l32, kk * 2 + half);
            const auto b = stage_frag<T>(sE, l32, kk * 2 + half);
            s = Elem<T>::mfma(a, b, s);
          }
          __syncthreads();
        }
      }

      // ---- dz, filter per 32 x 32 sub-tile ---------------------------------------------------------
      {
        const bool big = block_epilogue<T>(p, s, sCid + wave * 32, half, meta.lse2[l32], meta.g[l32], meta.h[l32],
                                           meta.tgt[l32]);
        const bool survives = (p.filter_eps < 0.0f) || (__ballot(big) != 0ull);
        const bool live = (static_cast<int64_t>(vc) * 128 + wave * 32 < p.v);
        const bool use = live && (survives || !p.filter_e);
        if (use) {
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const int cls = wave * 32 + 8 * r4 + 4 * half;
            uint2 pk;
            pk.x = static_cast<uint32_t>(Elem<T>::from_float(s[r4 * 4 + 0])) |
                   (static_cast<uint32_t>(Elem<T>::from_float(s[r4 * 4 + 1])) << 16);
            pk.y = static_cast<uint32_t>(Elem<T>::from_float(s[r4 * 4 + 2])) |
                   (static_cast<uint32_t>(Elem<T>::from_float(s[r4 * 4 + 3])) << 16);
            *reinterpret_cast<uint2*>(sDz + l32 * 256 + ((((cls >> 3) ^ (l32 & 7)) << 4) | ((cls & 7) << 1))) = pk;
          }
          if (lane == 0) atomicOr(&sMisc[1], 1 << wave);
        }
        if (lane == 0 && live && survives) {
          const int vg = vc * 4 + wave;
          atomicOr(&sBits[vg >> 5], 1u << (vg & 31));
        }
        if (lane == 0 && live) n_recomputed += 1;
      }
      __syncthreads();
      const uint32_t mask = static_cast<uint32_t>(sMisc[1]);
      if (!write_de || mask == 0u) continue;
      if (tid == 0) n_product += __popc(mask);

      // ---- dE^T (D x 32 rows) += C_cell^T . dz^T, 256 columns of D per stage ---------------------------
      typename Elem<T>::vec8 bz[8];
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        const uint4 v = *reinterpret_cast<const uint4*>(sDz + l32 * 256 + (((kk * 2 + half) ^ (l32 & 7)) << 4));
        bz[kk] = __builtin_bit_cast(typename Elem<T>::vec8, v);
      }
      {
        StageLoader<128, ALIGNED> lc;
        lc.load(sCid, p.c, p.stride_cv, p.stride_cd, d_begin, d_end, mask);
#pragma unroll
        for (int ci = 0; ci < kMaxChunks; ++ci) {
          if (ci < nchunks) {
            lc.store(sC, mask);
            __syncthreads();
            if (ci + 1 < nchunks)
              lc.load(sCid, p.c, p.stride_cv, p.stride_cd, d_begin + (ci + 1) * kStageCols, d_end, mask);
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
              if ((mask >> (kk >> 1)) & 1u) {
#pragma unroll
                for (int hb = 0; hb < 2; ++hb) {
                  const auto a = stage_frag_transposed<T>(sC, kk * 16 + half * 8, hb * 128 + wave * 32 + l32);
                  acc[ci][hb] = Elem<T>::mfma(a, bz[kk], acc[ci][hb]);
                }
              }
            }
            __syncthreads();
          }
        }
      }
    }
  }

  // ---- write the rows of this group, the bit row and the counters --------------------------------
  if (write_de) {
    const int row = meta.row[l32];
    if (row >= 0) {
#pragma unroll
      for (int ci = 0; ci < kMaxChunks; ++ci) {
        if (ci < nchunks) {
#pragma unroll
          for (int hb = 0; hb < 2; ++hb)
            store_rows<T>(acc[ci][hb], p.d_e, p.de_fp32 != 0, p.vec_e != 0, static_cast<int64_t>(row) * p.stride_e, 1,
                          d_begin + ci * kStageCols + hb * 128 + wave * 32, half, d_end);
        }
      }
    }
  }
  if (slice == 0) {
    if (p.kept_bits != nullptr)
      for (int w = tid; w < p.bit_words; w += kBwdThreads)
        p.kept_bits[static_cast<int64_t>(tg) * p.bit_words + w] = sBits[w];
    if (p.counters != nullptr) {
      // every wave counted the sub-tiles it recomputed; thread 0 those that entered a product
      if (lane == 0 && n_recomputed) atomicAdd(p.counters + 1, n_recomputed);
      if (tid == 0 && n_product) atomicAdd(p.counters + 2, n_product);
      if (tid == 0 && blockIdx.x == 0)
        atomicAdd(p.counters + 0, static_cast<unsigned long long>(p.ntg) * static_cast<unsigned long long>(p.nvg));
    }
  }
}

// ---------------------------------------------------------------------------------------------
// dC / dBias: workgroup = (class group of 32, slice of D)
// ---------------------------------------------------------------------------------------------
constexpr int kDcOffC = 0;                   // 16 KB  C stage: 32 classes x 256 columns
constexpr int kDcOffE = 16 * 1024;           // 16 KB  E stage: 32 rows x 256 columns
constexpr int kDcOffPart = 32 * 1024;        // 16 KB  partial logits of the four K quarters
constexpr int kDcOffDz = 48 * 1024;          //  2 KB  dz [class][row], 64 bytes per row
constexpr int kDcOffList = 50 * 1024;        // 16 KB  row-group list
constexpr int kDcOffMeta = 66 * 1024;
constexpr int kDcLdsBytes = kDcOffMeta + 5 * 128 + 128 + 128 + 64;

template <typename T, bool ALIGNED>
__global__ __launch_bounds__(kBwdThreads, 1) void bwd_dc_kernel(BwdParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sC = smem + kDcOffC;
  unsigned char* sE = smem + kDcOffE;
  float* sPart = reinterpret_cast<float*>(smem + kDcOffPart);
  unsigned char* sDz = smem + kDcOffDz;
  int* sList = reinterpret_cast<int*>(smem + kDcOffList);
  RowMeta meta;
  meta.row = reinterpret_cast<int*>(smem + kDcOffMeta);
  meta.tgt = meta.row + 32;
  meta.lse2 = reinterpret_cast<float*>(meta.tgt + 32);
  meta.g = meta.lse2 + 32;
  meta.h = meta.g + 32;
  int* sCid = reinterpret_cast<int*>(meta.h + 32);     // [32]
  float* sDb = reinterpret_cast<float*>(sCid + 32);    // [32] dBias of the group
  int* sMisc = reinterpret_cast<int*>(sDb + 32);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int vg = blockIdx.x / p.nslices;
  const int slice = blockIdx.x % p.nslices;
  const int d_begin = slice * p.dslice;
  const int d_end = min(static_cast<int>(p.d), d_begin + p.dslice);
  const int nchunks = (d_end - d_begin + kStageCols - 1) / kStageCols;
  const int D = static_cast<int>(p.d);
  const bool write_dc = (p.d_c != nullptr);
  const bool use_bits = (p.filter_c != 0);

  if (tid < 32) {
    const int64_t pos = static_cast<int64_t>(vg) * 32 + tid;
    int cid = -1;
    if (pos < p.v) cid = p.vocab_order ? p.vocab_order[pos] : static_cast<int>(pos);
    sCid[tid] = cid;
    sDb[tid] = 0.0f;
  }
  __syncthreads();

  f32x16 acc[kMaxChunks][2];
#pragma unroll
  for (int ci = 0; ci < kMaxChunks; ++ci)
#pragma unroll
    for (int hb = 0; hb < 2; ++hb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ci][hb][r] = 0.0f;
  unsigned long long n_product = 0;
  bool touched = false;

  for (int seg = 0; seg < p.ntg; seg += kListCap) {
    const int seg_n = min(kListCap, p.ntg - seg);
    if (use_bits) {
      if (wave == 0) {
        int n = 0;
        for (int base = 0; base < seg_n; base += 64) {
          bool f = false;
          if (base + lane < seg_n) {
            const uint32_t w = p.kept_bits[static_cast<int64_t>(seg + base + lane) * p.bit_words + (vg >> 5)];
            f = ((w >> (vg & 31)) & 1u) != 0u;
          }
          const unsigned long long m = __ballot(f);
          if (f) sList[n + __popcll(m & ((1ull << lane) - 1ull))] = seg + base + lane;
          n += __popcll(m);
        }
        if (lane == 0) sMisc[0] = n;
      }
      __syncthreads();
    }
    const int list_n = use_bits ? sMisc[0] : seg_n;

    for (int li = 0; li < list_n; ++li) {
      const int tg = use_bits ? sList[li] : seg + li;
      if (tid < 32) load_row_meta(p, static_cast<int64_t>(tg) * 32 + tid, tid, meta);
      __syncthreads();

      // ---- logits^T (32 classes x 32 rows): the 4 waves split every stage 4 ways along K ------------
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.0f;
      {
        StageLoader<32, ALIGNED> lc, le;
        const int nstages = (D + kStageCols - 1) / kStageCols;
        lc.load(sCid, p.c, p.stride_cv, p.stride_cd, 0, D, 0x1u);
        le.load(meta.row, p.e, p.stride_e, 1, 0, D, 0x1u);
        for (int st = 0; st < nstages; ++st) {
          lc.store(sC, 0x1u);
          le.store(sE, 0x1u);
          __syncthreads();
          if (st + 1 < nstages) {
            lc.load(sCid, p.c, p.stride_cv, p.stride_cd, (st + 1) * kStageCols, D, 0x1u);
            le.load(meta.row, p.e, p.stride_e, 1, (st + 1) * kStageCols, D, 0x1u);
          }
#pragma unroll
          for (int k4 = 0; k4 < 4; ++k4) {
            const int kk = wave * 4 + k4;
            const auto a = stage_frag<T>(sC, l32, kk * 2 + half);
            const auto b = stage_frag<T>(sE, l32, kk * 2 + half);
            s = Elem<T>::mfma(a, b, s);
          }
          __syncthreads();
        }
      }
      if (wave != 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) sPart[(wave * 16 + r) * 64 + lane] = s[r];
      }
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int w = 1; w < 4; ++w)
#pragma unroll
          for (int r = 0; r < 16; ++r) s[r] += sPart[(w * 16 + r) * 64 + lane];
        block_epilogue<T>(p, s, sCid, half, meta.lse2[l32], meta.g[l32], meta.h[l32], meta.tgt[l32]);
        // dz [class][row] for the dC product; row sums for dBias
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int cls = 8 * (r >> 2) + 4 * half + (r & 3);
          *reinterpret_cast<uint16_t*>(sDz + cls * 64 + l32 * 2) = Elem<T>::from_float(s[r]);
          float colsum = s[r];
#pragma unroll
          for (int off = 16; off >= 1; off >>= 1) colsum += __shfl_xor(colsum, off, 64);
          if (l32 == 0) sDb[cls] += colsum;
        }
      }
      __syncthreads();
      touched = true;
      if (tid == 0) n_product += 1;
      if (!write_dc) continue;

      // ---- dC^T (D x 32 classes) += E_group^T . dz, 256 columns of D per stage -----------------------------
      typename Elem<T>::vec8 bz[2];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const uint4 v = *reinterpret_cast<const uint4*>(sDz + l32 * 64 + ((kk * 2 + half) << 4));
        bz[kk] = __builtin_bit_cast(typename Elem<T>::vec8, v);
      }
      {
        StageLoader<32, ALIGNED> le;
        le.load(meta.row, p.e, p.stride_e, 1, d_begin, d_end, 0x1u);
#pragma unroll
        for (int ci = 0; ci < kMaxChunks; ++ci) {
          if (ci < nchunks) {
            le.store(sE, 0x1u);
            __syncthreads();
            if (ci + 1 < nchunks) le.load(meta.row, p.e, p.stride_e, 1, d_begin + (ci + 1) * kStageCols, d_end, 0x1u);
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
              for (int hb = 0; hb < 2; ++hb) {
                const auto a = stage_frag_transposed<T>(sE, kk * 16 + half * 8, hb * 128 + wave * 32 + l32);
                acc[ci][hb] = Elem<T>::mfma(a, bz[kk], acc[ci][hb]);
              }
            }
            __syncthreads();
          }
        }
      }
    }
  }

  // Rows nobody touched keep the caller's zeros.
  if (write_dc && touched) {
    const int cid = sCid[l32];
    if (cid >= 0) {
#pragma unroll
      for (int ci = 0; ci < kMaxChunks; ++ci) {
        if (ci < nchunks) {
#pragma unroll
          for (int hb = 0; hb < 2; ++hb)
            store_rows<T>(acc[ci][hb], p.d_c, p.dc_fp32 != 0, p.vec_c != 0, static_cast<int64_t>(cid) * p.stride_cv,
                          p.stride_cd, d_begin + ci * kStageCols + hb * 128 + wave * 32, half, d_end);
        }
      }
    }
  }
  if (slice == 0) {
    if (p.d_bias != nullptr && touched && tid < 32 && sCid[tid] >= 0) p.d_bias[sCid[tid]] = sDb[tid];
    if (p.counters != nullptr && tid == 0 && n_product) atomicAdd(p.counters + 3, n_product);
  }
}

}  // namespace cce

using namespace cce;

static int64_t bit_words_for(int64_t v) { return ((v + 31) / 32 + 31) / 32; }

extern "C" int64_t cce_backward_workspace_bytes(int64_t b, int64_t v, int64_t d) {
  (void)d;
  if (b <= 0 || v <= 0) return 0;
  return ((b + 31) / 32) * bit_words_for(v) * 4;
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
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (b < 0 || v <= 0 || d <= 0 || n_rows < 0 || shift < 0) return CCE_ERR_INVALID_ARGUMENT;
  if (b == 0) return CCE_OK;
  if (e == nullptr || c == nullptr || lse == nullptr || d_out == nullptr || targets == nullptr)
    return CCE_ERR_INVALID_ARGUMENT;
  if (valids == nullptr && b > n_rows) return CCE_ERR_INVALID_ARGUMENT;
  if (n_rows >= (int64_t(1) << 31) || v >= (int64_t(1) << 31) - 512 || d > (1 << 24)) return CCE_ERR_INVALID_ARGUMENT;
  if (dtype != CCE_DTYPE_BF16 && dtype != CCE_DTYPE_F16) return CCE_ERR_UNSUPPORTED_DTYPE;
  if (d_e == nullptr && d_c == nullptr && d_bias == nullptr) return CCE_OK;
  if (bit_words_for(v) > kDeMaxBitWords) return CCE_ERR_INVALID_ARGUMENT;

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
  // a bound just under eps keeps the cell: a little slack costs a recompute, never an error
  p.log_eps = (filtering && filter_eps > 0.0f) ? logf(filter_eps) - 0.01f : -INFINITY;
  p.d_out_is_scalar = d_out_is_scalar;
  p.de_fp32 = d_e_is_fp32;
  p.dc_fp32 = d_c_is_fp32;
  p.ntg = static_cast<int>((b + 31) / 32);
  p.nvc = static_cast<int>((v + 127) / 128);
  p.nvg = static_cast<int>((v + 31) / 32);
  p.bit_words = static_cast<int>(bit_words_for(v));
  p.nslices = static_cast<int>((d + kMaxChunks * kStageCols - 1) / (kMaxChunks * kStageCols));
  const int64_t per = (d + p.nslices - 1) / p.nslices;
  p.dslice = static_cast<int>((per + kStageCols - 1) / kStageCols * kStageCols);
  p.stat_cols = static_cast<int>((v + CCE_STAT_COLS - 1) / CCE_STAT_COLS);
  p.vec_e = (d_e != nullptr && stride_e % 4 == 0 && d % 4 == 0 && aligned16(d_e)) ? 1 : 0;
  p.vec_c = (d_c != nullptr && stride_cv % 4 == 0 && d % 4 == 0 && stride_cd == 1 && aligned16(d_c)) ? 1 : 0;
  p.sc = make_softcap(softcap);

  // The row-group kernel runs when dE is wanted, and also when only its survivor bits are (dC or
  // dBias filtered); it then skips the products.
  const bool need_dc_pass = (d_c != nullptr) || (d_bias != nullptr);
  const bool need_bits = need_dc_pass && p.filter_c;
  const bool need_de_pass = (d_e != nullptr) || need_bits;
  p.kept_bits = nullptr;
  if (need_bits) {
    const int64_t need = cce_backward_workspace_bytes(b, v, d);
    if (workspace == nullptr || workspace_bytes < need) return CCE_ERR_WORKSPACE_TOO_SMALL;
    if ((reinterpret_cast<uintptr_t>(workspace) & 3u) != 0) return CCE_ERR_MISALIGNED;
    p.kept_bits = static_cast<uint32_t*>(workspace);
  }
  // Cells may be skipped unseen only if a filtered sub-tile feeds nothing this pass produces.
  p.shortcut = (tile_max != nullptr && vocab_order == nullptr && filtering && filter_eps > 0.0f &&
                (d_e == nullptr || p.filter_e)) ? 1 : 0;

  const bool aligned = aligned16(e) && aligned16(c) && (d % 8 == 0) && (stride_e % 8 == 0) &&
                       (stride_cv % 8 == 0) && (stride_cd == 1);
  hipError_t err;
#define CCE_LAUNCH(KERN, LDS, GRID)                                                                 \
  do {                                                                                              \
    auto kern = KERN;                                                                               \
    err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                  \
                              hipFuncAttributeMaxDynamicSharedMemorySize, LDS);                     \
    if (err != hipSuccess) return status_from_hip(err);                                             \
    hipLaunchKernelGGL(kern, dim3(GRID), dim3(kBwdThreads), LDS, stream, p);                                \
  } while (0)
  if (need_de_pass) {
    const unsigned grid = static_cast<unsigned>(p.ntg) * static_cast<unsigned>(d_e != nullptr ? p.nslices : 1);
    BwdParams q = p;
    if (d_e == nullptr) { q.nslices = 1; q.dslice = p.dslice; }
    p = q;
    if (dtype == CCE_DTYPE_BF16) {
      if (aligned) CCE_LAUNCH((bwd_de_kernel<BF16, true>), kDeLdsBytes, grid);
      else CCE_LAUNCH((bwd_de_kernel<BF16, false>), kDeLdsBytes, grid);
    } else {
      if (aligned) CCE_LAUNCH((bwd_de_kernel<F16, true>), kDeLdsBytes, grid);
      else CCE_LAUNCH((bwd_de_kernel<F16, false>), kDeLdsBytes, grid);
    }
    err = hipGetLastError();
    if (err != hipSuccess) return status_from_hip(err);
  }
  if (need_dc_pass) {
    p.nslices = (d_c != nullptr) ? static_cast<int>((d + kMaxChunks * kStageCols - 1) / (kMaxChunks * kStageCols)) : 1;
    const unsigned grid = static_cast<unsigned>(p.nvg) * static_cast<unsigned>(p.nslices);
    if (dtype == CCE_DTYPE_BF16) {
      if (aligned) CCE_LAUNCH((bwd_dc_kernel<BF16, true>), kDcLdsBytes, grid);
      else CCE_LAUNCH((bwd_dc_kernel<BF16, false>), kDcLdsBytes, grid);
    } else {
      if (aligned) CCE_LAUNCH((bwd_dc_kernel<F16, true>), kDcLdsBytes, grid);
      else CCE_LAUNCH((bwd_dc_kernel<F16, false>), kDcLdsBytes, grid);
    }
  }
#undef CCE_LAUNCH
  return status_from_hip(hipGetLastError());
}
