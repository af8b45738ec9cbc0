// cce_backward: recompute logit tiles, form softmax - one-hot, filter, accumulate dE / dC / dBias
// on gfx950 -- without a single global atomic on the gradients.
//
// Global read-modify-write is the slow path of this chip (a few hundred G lane-updates/s), so the
// two gradients are produced by two ownership kernels whose accumulators never leave registers:
//
//   dE pass   one workgroup (4 waves) owns 32 valid rows (a "row group") and up to 2304 columns of dE.
//             It walks the 32-class sub-blocks of the vocabulary that can matter for its rows, four at a
//             time, recomputes their logits with MFMA, forms dz, applies the gradient filter per
//             32 x 32 sub-tile, and accumulates dE^T (D x 32 rows) += C_cell^T . dz^T in fp32 registers.
//             The rows are written once at the end.  It also records, one bit per 32 x 32 sub-tile,
//             which sub-tiles survived the filter.
//   dC pass   one workgroup owns 32 classes (and up to 2304 columns of dC), walks the row groups whose
//             bit is set (all of them when dC is not filtered), four at a time, recomputes the 32 x 32
//             logits, and accumulates dC^T (D x 32 classes) += E_cell^T . dz; dBias is the row sum of the
//             same dz.  Rows are written once at the end.
// Both passes are one kernel template with the roles of E and C swapped: bwd_owner_kernel for any layout,
// bwd_owner_fast_kernel (direct-to-LDS loads, D % 128 == 0, 16-byte aligned rows) for the common one.
//
// Which sub-blocks can matter: the forward pass left, per 32 rows x 32 classes, the largest
// soft-capped logit.  If the bound exp(cell_max - min_row lse) of a sub-block is below filter_eps, every
// |p| in it is below filter_eps, so it can survive the filter only if it holds a target of one of the
// rows: the others are skipped without being recomputed.
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
  int light_on;  // dC pass: class groups with at most kFLightMaxEntries entries are left to the light variant
  int* heavy_list;  // [1 + nvg]: count, then the class groups the light variant leaves to the full one
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
template <typename T, bool CAP, bool HAS_BIAS>
__device__ __forceinline__ bool block_epilogue_impl(const BwdParams& p, f32x16& acc, const int* cid32, int half,
                                                    float lse2, float g, float h, int tgt) {
  bool big = false;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int cid = cid32[8 * (r >> 2) + 4 * half + (r & 3)];
    float x = acc[r];
    if (HAS_BIAS) x += (cid >= 0) ? Elem<T>::to_float(p.bias[cid]) : 0.0f;
    float s2, damp = 1.0f;
    if (CAP) {
      const float t = __builtin_amdgcn_exp2f(x * p.sc.in_scale);
      const float w = __builtin_amdgcn_rcpf(1.0f + t);
      const float th = 1.0f - 2.0f * w;
      s2 = p.sc.out_scale * th;
      damp = 1.0f - th * th;
    } else {
      s2 = x * kLog2e;
    }
    const float pr = (cid >= 0) ? __builtin_amdgcn_exp2f(s2 - lse2) : 0.0f;
    const bool hit = (cid >= 0) && (cid == tgt);
    const float f = pr - (hit ? 1.0f : 0.0f);
    big = big || (fabsf(f) >= p.filter_eps);
    float dz = pr * (g + h) - (hit ? g : 0.0f);
    if (CAP) dz *= damp;
    acc[r] = dz;
  }
  return big;
}

// One uniform branch per block: each arm is straight-line code over the 16 values of a lane.
template <typename T>
__device__ __forceinline__ bool block_epilogue(const BwdParams& p, f32x16& acc, const int* cid32, int half,
                                               float lse2, float g, float h, int tgt) {
  if (p.bias != nullptr) {
    if (p.sc.on) return block_epilogue_impl<T, true, true>(p, acc, cid32, half, lse2, g, h, tgt);
    return block_epilogue_impl<T, false, true>(p, acc, cid32, half, lse2, g, h, tgt);
  }
  if (p.sc.on) return block_epilogue_impl<T, true, false>(p, acc, cid32, half, lse2, g, h, tgt);
  return block_epilogue_impl<T, false, false>(p, acc, cid32, half, lse2, g, h, tgt);
}

// ---------------------------------------------------------------------------------------------
// The ownership kernel, instantiated twice.
//
//   IS_DE = true   the workgroup owns 32 valid rows ("own" side = rows of E) and walks class
//                  sub-blocks of 32 ("other" side = rows of C); it writes dE rows and the survivor
//                  bits.
//   IS_DE = false  the workgroup owns 32 classes (own = rows of C) and walks row groups of 32
//                  (other = rows of E); it writes dC rows and dBias.
//
// Four list entries are processed per trip as one "virtual cell" of 128 other-side rows gathered by
// id (the entries need not be neighbours): wave w recomputes the 32 x 32 logits of entry w against
// the own rows over all of D, forms dz, and then all four waves accumulate
//     own_grad^T (D x 32 own) += Other_cell^T (D x 128) . dz (128 x 32 own)
// with wave w owning the 32-column blocks w and w + 4 of every 256 columns of D.
// ---------------------------------------------------------------------------------------------
constexpr int kOffOther = 0;                      // 64 KB  other-side stage: 128 rows x 256 columns
constexpr int kOffOwn = 64 * 1024;                // 16 KB  own-side stage: 32 rows x 256 columns
constexpr int kOffDz = 80 * 1024;                 //  8 KB  dz [own][other], 256 bytes per own row
constexpr int kOffList = 88 * 1024;               // 16 KB  entry list
constexpr int kOffFlag = 104 * 1024;              //  1 KB  per-cell sub-block masks (dE)
constexpr int kOffBits = 105 * 1024;              //  8 KB  survivor-bit row (dE)
constexpr int kMaxBitWords = 2048;                //        (V <= 2 M classes)
constexpr int kOffMeta = kOffBits + kMaxBitWords * 4;
constexpr int kMetaRows = 128;
constexpr int kBwdLdsBytes = kOffMeta + 5 * kMetaRows * 4 + 32 * 4 + 128 * 4 + 128 * 4 + 64;
constexpr int kSegCells = 1024;                   // dE: 128-class cells scanned per pass (<= 4096 entries)

template <typename T, bool ALIGNED, bool IS_DE>
__global__ __launch_bounds__(kBwdThreads, 1) void bwd_owner_kernel(BwdParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sOther = smem + kOffOther;
  unsigned char* sOwn = smem + kOffOwn;
  unsigned char* sDz = smem + kOffDz;
  int* sList = reinterpret_cast<int*>(smem + kOffList);
  unsigned char* sFlag = smem + kOffFlag;
  uint32_t* sBits = reinterpret_cast<uint32_t*>(smem + kOffBits);
  RowMeta meta;  // per token row: 32 own rows (dE) or the 128 rows of the current virtual cell (dC)
  meta.row = reinterpret_cast<int*>(smem + kOffMeta);
  meta.tgt = meta.row + kMetaRows;
  meta.lse2 = reinterpret_cast<float*>(meta.tgt + kMetaRows);
  meta.g = meta.lse2 + kMetaRows;
  meta.h = meta.g + kMetaRows;
  int* sOwnCid = reinterpret_cast<int*>(meta.h + kMetaRows);  // [32]  dC: class ids of the own rows
  int* sCellCid = sOwnCid + 32;                                // [128] dE: class ids of the virtual cell
  float* sDb = reinterpret_cast<float*>(sCellCid + 128);       // [4][32] dC: per-wave dBias of the own classes
  int* sMisc = reinterpret_cast<int*>(sDb + 128);               // [0] list length, [1] entry mask, [2] min lse

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int own = blockIdx.x / p.nslices;  // row group (dE) or class group (dC)
  const int slice = blockIdx.x % p.nslices;
  const int d_begin = slice * p.dslice;
  const int d_end = min(static_cast<int>(p.d), d_begin + p.dslice);
  const int nchunks = (d_end - d_begin + kStageCols - 1) / kStageCols;
  const int D = static_cast<int>(p.d);
  const bool write_out = IS_DE ? (p.d_e != nullptr) : (p.d_c != nullptr);

  // ---- own-side metadata -----------------------------------------------------------------------
  float my_lse = INFINITY;
  if (IS_DE) {
    if (tid < 32) my_lse = load_row_meta(p, static_cast<int64_t>(own) * 32 + tid, tid, meta);
    if (wave == 0) {
      const float mn = wave_min(my_lse);
      if (lane == 0) reinterpret_cast<float*>(sMisc)[2] = mn;
    }
    for (int w = tid; w < p.bit_words; w += kBwdThreads) sBits[w] = 0u;
  } else if (tid < 32) {
    const int64_t pos = static_cast<int64_t>(own) * 32 + tid;
    int cid = -1;
    if (pos < p.v) cid = p.vocab_order ? p.vocab_order[pos] : static_cast<int>(pos);
    sOwnCid[tid] = cid;
#pragma unroll
    for (int w = 0; w < 4; ++w) sDb[w * 32 + tid] = 0.0f;
  }
  __syncthreads();
  const float min_lse = reinterpret_cast<float*>(sMisc)[2];
  const int* own_ids = IS_DE ? meta.row : sOwnCid;

  // wave w owns columns [32 w, 32 w + 32) and [128 + 32 w, 128 + 32 w + 32) of every 256-column chunk
  f32x16 acc[kMaxChunks][2];
#pragma unroll
  for (int ci = 0; ci < kMaxChunks; ++ci)
#pragma unroll
    for (int hb = 0; hb < 2; ++hb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[ci][hb][r] = 0.0f;

  unsigned long long n_recomputed = 0, n_product = 0;
  bool touched = false;
  const bool use_list = IS_DE ? (p.shortcut != 0) : (p.filter_c != 0);
  const int n_units = IS_DE ? p.nvc : p.ntg;          // what a pass scans: cells (dE) or row groups (dC)
  const int seg_units = IS_DE ? kSegCells : kListCap;

  for (int seg = 0; seg < n_units; seg += seg_units) {
    const int seg_n = min(seg_units, n_units - seg);
    // ---- entries of this pass: class sub-blocks (dE) or row groups (dC), in increasing order --------
    if (use_list) {
      if (IS_DE) {
        // a cell whose bound reaches eps needs all four sub-blocks; otherwise only those holding a target
        for (int j = tid; j < seg_n; j += kBwdThreads) {
          // one bound per 32-class sub-block: exp(max logit - min lse of the 32 rows) against eps
          const float* cell = p.tile_max + static_cast<int64_t>(own) * p.stat_cols + static_cast<int64_t>(seg + j) * 4;
          const int nsb = min(4, p.stat_cols - (seg + j) * 4);
          int m = 0;
#pragma unroll
          for (int sb = 0; sb < 4; ++sb)
            if (sb < nsb && cell[sb] - min_lse >= p.log_eps) m |= 1 << sb;
          sFlag[j] = static_cast<unsigned char>(m);
        }
        __syncthreads();
        if (tid < 32) {
          const int t = meta.tgt[tid];
          if (t >= 0) {
            const int cell = t / 128 - seg;
            if (cell >= 0 && cell < seg_n)
              atomicOr(reinterpret_cast<unsigned int*>(sFlag) + (cell >> 2), (1u << ((t >> 5) & 3)) << ((cell & 3) * 8));
          }
        }
        __syncthreads();
      }
      if (wave == 0) {  // ordered compaction: the accumulation order, hence the result, is fixed
        int n = 0;
        for (int base = 0; base < seg_n; base += 64) {
          if (IS_DE) {
            const int m = (base + lane < seg_n) ? sFlag[base + lane] : 0;
            const int cnt = __popc(m);
            int incl = cnt;  // inclusive prefix sum over the wave
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
              const int v = __shfl_up(incl, off, 64);
              if (lane >= off) incl += v;
            }
            int pos = n + incl - cnt;
#pragma unroll
            for (int sb = 0; sb < 4; ++sb)
              if ((m >> sb) & 1) sList[pos++] = (seg + base + lane) * 4 + sb;
            n += __shfl(incl, 63, 64);
          } else {
            bool f = false;
            if (base + lane < seg_n) {
              const uint32_t w = p.kept_bits[static_cast<int64_t>(seg + base + lane) * p.bit_words + (own >> 5)];
              f = ((w >> (own & 31)) & 1u) != 0u;
            }
            const unsigned long long m = __ballot(f);
            if (f) sList[n + __popcll(m & ((1ull << lane) - 1ull))] = seg + base + lane;
            n += __popcll(m);
          }
        }
        if (lane == 0) sMisc[0] = n;
      }
      __syncthreads();
    }
    const int list_n = use_list ? sMisc[0] : (IS_DE ? seg_n * 4 : seg_n);

    for (int li = 0; li < list_n; li += 4) {
      // ---- the virtual cell: up to four entries, 32 other-side rows each -------------------------------
      if (IS_DE) {
        if (tid < 128) {
          const int k = li + (tid >> 5);
          int cid = -1;
          if (k < list_n) {
            const int vg = use_list ? sList[k] : seg * 4 + k;
            const int64_t pos = static_cast<int64_t>(vg) * 32 + (tid & 31);
            if (pos < p.v) cid = p.vocab_order ? p.vocab_order[pos] : static_cast<int>(pos);
          }
          sCellCid[tid] = cid;
        }
      } else {
        if (tid < 128) {
          const int k = li + (tid >> 5);
          int64_t i = p.b;  // no row
          if (k < list_n) i = static_cast<int64_t>(use_list ? sList[k] : seg + k) * 32 + (tid & 31);
          load_row_meta(p, i, tid, meta);
        }
      }
      if (tid == 0) sMisc[1] = 0;
      __syncthreads();
      const int* other_ids = IS_DE ? sCellCid : meta.row;
      const int entry = li + wave;
      const bool have_entry = entry < list_n;
      const int entry_id = have_entry ? (use_list ? sList[entry] : (IS_DE ? seg * 4 + entry : seg + entry)) : -1;

      // ---- logits^T of (entry of this wave) x (own rows) over all of D --------------------------------------
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.0f;
      {
        StageLoader<128, ALIGNED> lo;
        StageLoader<32, ALIGNED> lw;
        const uint16_t* other_base = IS_DE ? p.c : p.e;
        const uint16_t* own_base = IS_DE ? p.e : p.c;
        const int64_t other_sr = IS_DE ? p.stride_cv : p.stride_e;
        const int64_t other_sc = IS_DE ? p.stride_cd : 1;
        const int64_t own_sr = IS_DE ? p.stride_e : p.stride_cv;
        const int64_t own_sc = IS_DE ? 1 : p.stride_cd;
        const int nstages = (D + kStageCols - 1) / kStageCols;
        lo.load(other_ids, other_base, other_sr, other_sc, 0, D, 0xfu);
        lw.load(own_ids, own_base, own_sr, own_sc, 0, D, 0x1u);
        for (int st = 0; st < nstages; ++st) {
          lo.store(sOther, 0xfu);
          lw.store(sOwn, 0x1u);
          __syncthreads();
          if (st + 1 < nstages) {
            lo.load(other_ids, other_base, other_sr, other_sc, (st + 1) * kStageCols, D, 0xfu);
            lw.load(own_ids, own_base, own_sr, own_sc, (st + 1) * kStageCols, D, 0x1u);
          }
#pragma unroll
          for (int kk = 0; kk < 16; ++kk) {
            // MFMA A operand = class rows, B operand = token rows
            const auto fo = stage_frag<T>(sOther, wave * 32 + l32, kk * 2 + half);
            const auto fw = stage_frag<T>(sOwn, l32, kk * 2 + half);
            s = IS_DE ? Elem<T>::mfma(fo, fw, s) : Elem<T>::mfma(fw, fo, s);
          }
          __syncthreads();
        }
      }

      // ---- dz of this wave's 32 x 32 block (lane = token row, registers = classes) ----------------------------
      {
        const int mrow = IS_DE ? l32 : wave * 32 + l32;  // metadata slot of this lane's token row
        const int* cid32 = IS_DE ? sCellCid + wave * 32 : sOwnCid;
        const bool big = block_epilogue<T>(p, s, cid32, half, meta.lse2[mrow], meta.g[mrow], meta.h[mrow], meta.tgt[mrow]);
        bool use = have_entry;
        if (IS_DE) {
          const bool survives = (p.filter_eps < 0.0f) || (__ballot(big) != 0ull);
          const bool live = have_entry && (static_cast<int64_t>(entry_id) * 32 < p.v);
          use = live && (survives || !p.filter_e);
          if (lane == 0 && live && survives) atomicOr(&sBits[entry_id >> 5], 1u << (entry_id & 31));
          if (lane == 0 && live) n_recomputed += 1;
        }
        if (use) {
          if (IS_DE) {
            // dz [own row = lane][class of the cell]: four consecutive classes per store
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
              const int k = wave * 32 + 8 * r4 + 4 * half;
              uint2 pk;
              pk.x = Elem<T>::pack2(s[r4 * 4 + 0], s[r4 * 4 + 1]);
              pk.y = Elem<T>::pack2(s[r4 * 4 + 2], s[r4 * 4 + 3]);
              *reinterpret_cast<uint2*>(sDz + l32 * 256 + ((((k >> 3) ^ (l32 & 7)) << 4) | ((k & 7) << 1))) = pk;
            }
          } else {
            // dz [own class][row of the cell = lane]; row sums feed dBias
            const int k = wave * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int cls = 8 * (r >> 2) + 4 * half + (r & 3);
              *reinterpret_cast<uint16_t*>(sDz + cls * 256 + ((((k >> 3) ^ (cls & 7)) << 4) | ((k & 7) << 1))) =
                  Elem<T>::from_float(s[r]);
              if (p.d_bias != nullptr) {
                float colsum = s[r];
#pragma unroll
                for (int off = 16; off >= 1; off >>= 1) colsum += __shfl_xor(colsum, off, 64);
                if (l32 == 0) sDb[wave * 32 + cls] += colsum;  // one writer per slot: deterministic
              }
            }
          }
          if (lane == 0) atomicOr(&sMisc[1], 1 << wave);
        }
      }
      __syncthreads();
      const uint32_t mask = static_cast<uint32_t>(sMisc[1]);
      if (mask == 0u) continue;
      touched = true;
      if (tid == 0) n_product += __popc(mask);
      if (!write_out) continue;

      // ---- own_grad^T (D x 32) += Other_cell^T . dz, 256 columns of D per stage ------------------------------------
      typename Elem<T>::vec8 bz[8];
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        const uint4 v = *reinterpret_cast<const uint4*>(sDz + l32 * 256 + (((kk * 2 + half) ^ (l32 & 7)) << 4));
        bz[kk] = __builtin_bit_cast(typename Elem<T>::vec8, v);
      }
      {
        StageLoader<128, ALIGNED> lo;
        const uint16_t* other_base = IS_DE ? p.c : p.e;
        const int64_t other_sr = IS_DE ? p.stride_cv : p.stride_e;
        const int64_t other_sc = IS_DE ? p.stride_cd : 1;
        lo.load(other_ids, other_base, other_sr, other_sc, d_begin, d_end, mask);
#pragma unroll
        for (int ci = 0; ci < kMaxChunks; ++ci) {
          if (ci < nchunks) {
            lo.store(sOther, mask);
            __syncthreads();
            if (ci + 1 < nchunks) lo.load(other_ids, other_base, other_sr, other_sc, d_begin + (ci + 1) * kStageCols, d_end, mask);
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
              if ((mask >> (kk >> 1)) & 1u) {
#pragma unroll
                for (int hb = 0; hb < 2; ++hb) {
                  const auto a = stage_frag_transposed<T>(sOther, kk * 16 + half * 8, hb * 128 + wave * 32 + l32);
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

  // ---- write the own rows once: a row group nobody touched keeps the zeros dE came with; a class group
  // always writes its rows of dC (zeros when nothing survived for it), so dC need not be cleared beforehand
  if (write_out && (touched || !IS_DE)) {
    const int id = own_ids[l32];
    if (id >= 0) {
#pragma unroll
      for (int ci = 0; ci < kMaxChunks; ++ci) {
        if (ci < nchunks) {
#pragma unroll
          for (int hb = 0; hb < 2; ++hb) {
            const int col0 = d_begin + ci * kStageCols + hb * 128 + wave * 32;
            if (IS_DE)
              store_rows<T>(acc[ci][hb], p.d_e, p.de_fp32 != 0, p.vec_e != 0, static_cast<int64_t>(id) * p.stride_e, 1,
                            col0, half, d_end);
            else
              store_rows<T>(acc[ci][hb], p.d_c, p.dc_fp32 != 0, p.vec_c != 0, static_cast<int64_t>(id) * p.stride_cv,
                            p.stride_cd, col0, half, d_end);
          }
        }
      }
    }
  }
  if (slice == 0) {
    if (IS_DE) {
      if (p.kept_bits != nullptr)
        for (int w = tid; w < p.bit_words; w += kBwdThreads)
          p.kept_bits[static_cast<int64_t>(own) * p.bit_words + w] = sBits[w];
      if (p.counters != nullptr) {
        if (lane == 0 && n_recomputed) atomicAdd(p.counters + 1, n_recomputed);
        if (tid == 0 && n_product) atomicAdd(p.counters + 2, n_product);
        if (tid == 0 && blockIdx.x == 0)
          atomicAdd(p.counters + 0, static_cast<unsigned long long>(p.ntg) * static_cast<unsigned long long>(p.nvg));
      }
    } else {
      if (p.d_bias != nullptr && touched && tid < 32 && sOwnCid[tid] >= 0)
        p.d_bias[sOwnCid[tid]] = (sDb[tid] + sDb[32 + tid]) + (sDb[64 + tid] + sDb[96 + tid]);
      if (p.counters != nullptr && tid == 0 && n_product) atomicAdd(p.counters + 3, n_product);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Fast variant of the ownership kernel (16-byte aligned rows, unit column stride, D % 128 == 0):
// the same algorithm with direct global -> LDS loads (no staging registers, no LDS stores) through a
// ring of 128-column stages.  Both phases of a trip are bound by memory latency and gather
// bandwidth, not by the MFMAs, so what matters is how much is in flight and how little is fetched:
//   * a stage holds the rows of the entries that are present, then the own rows; a short trip has
//     small stages, so 3 (3-4 entries), 5 (2) or 7 (1) of them fit the 120 KB ring;
//   * the product phase fetches again only the entries whose dz is used;
//   * the transposed product operand comes from the LDS transpose read, two per fragment;
//   * all MFMAs are written as inline assembly with their accumulators pinned (16 chunks of the
//     gradient in the 256 accumulation registers, the rest and the logits in ordinary registers):
//     288 + 16 accumulator registers do not fit one file, and left alone the compiler spills;
//   * the gradient tile leaves through LDS as whole rows, 1 KB per row and store instruction.
//
// Stage layout: 256-byte rows (128 columns), 16-byte chunks XOR-swizzled with (row & 15); one load
// instruction of a wave fills 1 KB = 4 rows, lane l -> row (l >> 4), chunk slot (l & 15).  Other-side
// block b = q * 4 + wave holds rows [4 b, 4 b + 4) of the 128-row virtual cell; own-side likewise for
// its 32 rows.  A row id of -1 (no row: past the last valid row or the last class) is fetched from a
// line of zeros, whatever the stage: its products are exactly zero and no non-finite value of another
// row of the matrices can leak into real rows through it.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) uint16_t g_owner_zero_line[128];  // never written

constexpr int kFCols = 128;
constexpr int kFRowBytes = 256;
constexpr int kFOtherBytes = 128 * kFRowBytes;      // 32 KB
constexpr int kFOwnBytes = 32 * kFRowBytes;         //  8 KB
constexpr int kFStageBytes = kFOtherBytes + kFOwnBytes;
constexpr int kFMaxChunks = 18;                     // 18 * 128 = 2304 columns of D per workgroup
// LDS layout.  LIGHT (the dC pass of class groups with at most two entries, below): a 48 KB ring and no
// survivor-bit row, 68 KB in all, so that two workgroups share a compute unit.
template <bool LIGHT>
struct FastLds {
  static constexpr int kRing = LIGHT ? 48 * 1024 : 3 * kFStageBytes;  // 48 KB / 120 KB
  static constexpr int kOffDz = kRing;                   //   8 KB dz [own][other]
  static constexpr int kOffList = kOffDz + 8 * 1024;     //   8 KB entry list (2048 entries + 3 carried over)
  static constexpr int kOffFlag = kOffList + 8 * 1024 + 16;  // 512 B per-cell sub-block masks (dE)
  static constexpr int kOffBits = kOffFlag + 512;        //   8 KB survivor-bit row (dE)
  static constexpr int kOffMeta = kOffBits + (LIGHT ? 0 : kMaxBitWords * 4);
  static constexpr int kBytes = kOffMeta + 5 * kMetaRows * 4 + 32 * 4 + 128 * 4 + 128 * 4 + 64;
};
constexpr int kFLdsBytes = FastLds<false>::kBytes;
constexpr int kFLightLdsBytes = FastLds<true>::kBytes;
constexpr int kFLightMaxEntries = 2;
constexpr int kLightStores = 4;                     // store instructions per wave and 128-column chunk of the light dC pass                // entries of a class group the light dC pass takes on
constexpr int kFSegCells = 512;                     // dE: cells scanned per pass (<= 2048 entries)
constexpr int kFListCap = 2048;
static_assert(kFLdsBytes <= 160 * 1024 && 2 * kFLightLdsBytes <= 160 * 1024, "LDS budget of gfx950");

template <typename T>
__device__ __forceinline__ typename Elem<T>::vec8 fstage_frag(const unsigned char* lds, int row, int chunk) {
  const uint4 v = *reinterpret_cast<const uint4*>(lds + row * kFRowBytes + ((chunk ^ (row & 15)) << 4));
  return __builtin_bit_cast(typename Elem<T>::vec8, v);
}

typedef short short4_t __attribute__((ext_vector_type(4)));

// MFMA operand whose reduction index runs over the stage rows k0 + 8 (lane >> 5) .. + 7, for column
// col0 + (lane & 31): two LDS transpose reads (`ds_read_b64_tr_b16`) of four rows each.  In one such
// read a group of 16 lanes supplies 16 addresses of 4 elements -- lane i: row r0 + (i >> 2), columns
// m0 + 4 (i & 3) .. + 3 -- and lane i receives the elements [r0 .. r0 + 3][m0 + i].
template <typename T>
__device__ __forceinline__ typename Elem<T>::vec8 fstage_frag_transposed(const unsigned char* lds, int k0, int col0,
                                                                         int lane) {
  const int col = col0 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int ra = k0 + 8 * (lane >> 5) + ((lane >> 2) & 3);
  const int rb = ra + 4;
  const unsigned char* pa = lds + ra * kFRowBytes + ((((col >> 3) ^ (ra & 15)) << 4) | ((col & 7) << 1));
  const unsigned char* pb = lds + rb * kFRowBytes + ((((col >> 3) ^ (rb & 15)) << 4) | ((col & 7) << 1));
  struct {
    short4_t lo, hi;
  } v;
  v.lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(pa));
  v.hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(pb));
  return __builtin_bit_cast(typename Elem<T>::vec8, v);
}

// s_waitcnt vmcnt(n) for a wave-uniform n out of the values the rings below can ask for (the immediate must be a
// constant); anything else waits for everything, which is always safe.  The list is kept short: the product loop of
// the full variant is unrolled 18 times around it.
__device__ __forceinline__ void wait_vmcnt_upto(int n) {
  switch (n) {
    case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
    case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
    case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
    case 18: asm volatile("s_waitcnt vmcnt(18)" ::: "memory"); break;
    case 20: asm volatile("s_waitcnt vmcnt(20)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}
// ... and for any even n up to 30 (the light variant, whose product loop is not unrolled).
__device__ __forceinline__ void wait_vmcnt_upto_wide(int n) {
  switch (n) {
#define CCE_WAIT_CASE(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    CCE_WAIT_CASE(2) CCE_WAIT_CASE(4) CCE_WAIT_CASE(6) CCE_WAIT_CASE(8) CCE_WAIT_CASE(10) CCE_WAIT_CASE(12)
    CCE_WAIT_CASE(14) CCE_WAIT_CASE(16) CCE_WAIT_CASE(18) CCE_WAIT_CASE(20) CCE_WAIT_CASE(22) CCE_WAIT_CASE(24)
    CCE_WAIT_CASE(26) CCE_WAIT_CASE(28) CCE_WAIT_CASE(30)
#undef CCE_WAIT_CASE
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}

template <typename T, bool IS_DE, bool LIGHT = false>
__global__ __launch_bounds__(kBwdThreads, LIGHT ? 2 : 1) void bwd_owner_fast_kernel(BwdParams p) {
  static_assert(!(LIGHT && IS_DE), "the light variant is a dC pass");
  using Lds = FastLds<LIGHT>;
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sDz = smem + Lds::kOffDz;
  int* sList = reinterpret_cast<int*>(smem + Lds::kOffList);
  unsigned char* sFlag = smem + Lds::kOffFlag;
  uint32_t* sBits = reinterpret_cast<uint32_t*>(smem + Lds::kOffBits);
  RowMeta meta;
  meta.row = reinterpret_cast<int*>(smem + Lds::kOffMeta);
  meta.tgt = meta.row + kMetaRows;
  meta.lse2 = reinterpret_cast<float*>(meta.tgt + kMetaRows);
  meta.g = meta.lse2 + kMetaRows;
  meta.h = meta.g + kMetaRows;
  int* sOwnCid = reinterpret_cast<int*>(meta.h + kMetaRows);
  int* sCellCid = sOwnCid + 32;
  float* sDb = reinterpret_cast<float*>(sCellCid + 128);
  int* sMisc = reinterpret_cast<int*>(sDb + 128);
  const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(smem));

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int half = lane >> 5;
  int own = blockIdx.x / p.nslices;
  const int slice = blockIdx.x % p.nslices;
  if (IS_DE && blockIdx.x == 0 && threadIdx.x == 0 && p.heavy_list != nullptr) p.heavy_list[0] = 0;  // for the dC passes
  if (!IS_DE && !LIGHT && p.light_on) {
    // the full dC pass after the light one: only the class groups that one listed
    if (own >= p.heavy_list[0]) return;
    own = p.heavy_list[1 + own];
  }
  const int d_begin = slice * p.dslice;
  const int d_end = min(static_cast<int>(p.d), d_begin + p.dslice);
  const int nchunks = (d_end - d_begin) / kFCols;
  const int D = static_cast<int>(p.d);
  const int nstages = D / kFCols;
  const bool write_out = IS_DE ? (p.d_e != nullptr) : (p.d_c != nullptr);

  const uint16_t* other_base = IS_DE ? p.c : p.e;
  const uint16_t* own_base = IS_DE ? p.e : p.c;
  const int64_t other_sr = IS_DE ? p.stride_cv : p.stride_e;
  const int64_t own_sr = IS_DE ? p.stride_e : p.stride_cv;
  // element offset of the chunk this lane fetches inside a 128-column stage
  const int lane_chunk = ((lane & 15) ^ ((4 * wave + (lane >> 4)) & 15)) * 8;

  float my_lse = INFINITY;
  if (IS_DE) {
    if (tid < 32) my_lse = load_row_meta(p, static_cast<int64_t>(own) * 32 + tid, tid, meta);
    if (wave == 0) {
      const float mn = wave_min(my_lse);
      if (lane == 0) reinterpret_cast<float*>(sMisc)[2] = mn;
    }
    for (int w = tid; w < p.bit_words; w += kBwdThreads) sBits[w] = 0u;
  } else if (tid < 32) {
    const int64_t pos = static_cast<int64_t>(own) * 32 + tid;
    int cid = -1;
    if (pos < p.v) cid = p.vocab_order ? p.vocab_order[pos] : static_cast<int>(pos);
    sOwnCid[tid] = cid;
#pragma unroll
    for (int w = 0; w < 4; ++w) sDb[w * 32 + tid] = 0.0f;
  }
  __syncthreads();
  const float min_lse = reinterpret_cast<float*>(sMisc)[2];
  const int* own_ids = IS_DE ? meta.row : sOwnCid;

  // own-side load pointers (2 per wave and stage), fixed for the whole kernel
  // (a row that does not exist points at the line of zeros and does not advance with the stage)
  const uint16_t* zero_chunk = g_owner_zero_line + (lane & 15) * 8;
  const uint16_t* own_ptr[2];
  int own_step[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int id = own_ids[4 * (q * 4 + wave) + (lane >> 4)];
    own_ptr[q] = (id < 0) ? zero_chunk : own_base + static_cast<int64_t>(id) * own_sr + lane_chunk;
    own_step[q] = (id < 0) ? 0 : 1;
  }

  // wave w owns columns [32 w, 32 w + 32) of every 128-column chunk
  // (the light variant keeps no gradient between chunks: one trip at most, every chunk leaves as it is formed)
  constexpr int kAccChunks = LIGHT ? 1 : kFMaxChunks;
  f32x16 acc[kAccChunks];
#pragma unroll
  for (int ci = 0; ci < kAccChunks; ++ci)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[ci][r] = 0.0f;

  // light variant: the 32 own rows x 128 columns of one chunk, 16-bit, straight from the accumulator block of
  // this wave (lane = own row, registers = 4 x 4 consecutive columns)
  auto store_chunk_direct = [&](int ci, const f32x16& a) {
    const int id = own_ids[l32];
    if (id < 0) return;
    uint16_t* dst = static_cast<uint16_t*>(p.d_c) + static_cast<int64_t>(id) * own_sr + d_begin + ci * kFCols + wave * 32 + 4 * half;
    // exactly kLightStores store instructions per wave and chunk (the product loop below counts them: stores share
    // the counter its loads are awaited on), whatever the compiler would make of four plain assignments
#pragma unroll
    for (int r4 = 0; r4 < kLightStores; ++r4) {
      uint2 pk;
      pk.x = Elem<T>::pack2(a[r4 * 4 + 0], a[r4 * 4 + 1]);
      pk.y = Elem<T>::pack2(a[r4 * 4 + 2], a[r4 * 4 + 3]);
      asm volatile("global_store_dwordx2 %0, %1, off" ::"v"(dst + 8 * r4), "v"(pk) : "memory");
    }
  };

  unsigned long long n_recomputed = 0, n_product = 0;
  bool touched = false;
  const bool use_list = IS_DE ? (p.shortcut != 0) : (p.filter_c != 0);
  const int n_units = IS_DE ? p.nvc : p.ntg;
  const int seg_units = IS_DE ? kFSegCells : kFListCap;

  int carry = 0;  // listed entries a segment left over for the next one (trips are filled four at a time)
  for (int seg = 0; seg < n_units; seg += seg_units) {
    const int seg_n = min(seg_units, n_units - seg);
    if (use_list) {
      if (IS_DE) {
        for (int j = tid; j < seg_n; j += kBwdThreads) {
          // one bound per 32-class sub-block: exp(max logit - min lse of the 32 rows) against eps
          const float* cell = p.tile_max + static_cast<int64_t>(own) * p.stat_cols + static_cast<int64_t>(seg + j) * 4;
          const int nsb = min(4, p.stat_cols - (seg + j) * 4);
          int m = 0;
#pragma unroll
          for (int sb = 0; sb < 4; ++sb)
            if (sb < nsb && cell[sb] - min_lse >= p.log_eps) m |= 1 << sb;
          sFlag[j] = static_cast<unsigned char>(m);
        }
        __syncthreads();
        if (tid < 32) {
          const int t = meta.tgt[tid];
          if (t >= 0) {
            const int cell = t / 128 - seg;
            if (cell >= 0 && cell < seg_n)
              atomicOr(reinterpret_cast<unsigned int*>(sFlag) + (cell >> 2), (1u << ((t >> 5) & 3)) << ((cell & 3) * 8));
          }
        }
        __syncthreads();
      }
      if (wave == 0) {
        int n = carry;
        uint32_t kept_word[4] = {0u, 0u, 0u, 0u};
        for (int base = 0; base < seg_n; base += 64) {
          if (IS_DE) {
            const int m = (base + lane < seg_n) ? sFlag[base + lane] : 0;
            const int cnt = __popc(m);
            int incl = cnt;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
              const int v = __shfl_up(incl, off, 64);
              if (lane >= off) incl += v;
            }
            int pos = n + incl - cnt;
#pragma unroll
            for (int sb = 0; sb < 4; ++sb)
              if ((m >> sb) & 1) sList[pos++] = (seg + base + lane) * 4 + sb;
            n += __shfl(incl, 63, 64);
          } else {
            // four independent loads per lane, then four ballots: one round trip to memory per 256 row groups
            if ((base & 255) == 0) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const int u = base + j * 64 + lane;
                uint32_t w = 0u;
                if (u < seg_n) w = p.kept_bits[static_cast<int64_t>(seg + u) * p.bit_words + (own >> 5)];
                kept_word[j] = w;
              }
            }
            const bool f = ((kept_word[(base >> 6) & 3] >> (own & 31)) & 1u) != 0u;
            const unsigned long long m = __ballot(f);
            if (f) sList[n + __popcll(m & ((1ull << lane) - 1ull))] = seg + base + lane;
            n += __popcll(m);
          }
        }
        if (lane == 0) sMisc[0] = n;
      }
      __syncthreads();
    }
    const int list_n = use_list ? sMisc[0] : (IS_DE ? seg_n * 4 : seg_n);
    // Class groups with few entries belong to the light variant when it runs (p.light_on, one segment only).
    if (LIGHT && list_n > kFLightMaxEntries) {
      if (tid == 0) p.heavy_list[1 + atomicAdd(p.heavy_list, 1)] = own;
      return;
    }
    // A class group nothing survived for goes straight to writing its zeros.
    if (!IS_DE && list_n == 0 && n_units <= seg_units) break;
    // Only the last segment runs a trip that is not full: what is left over goes to the front of the next list.
    const bool keep_rest = use_list && (seg + seg_units < n_units);
    const int run_n = keep_rest ? (list_n & ~3) : list_n;

    for (int li = 0; li < run_n; li += 4) {
      if (IS_DE) {
        if (tid < 128) {
          const int k = li + (tid >> 5);
          int cid = -1;
          if (k < list_n) {
            const int vg = use_list ? sList[k] : seg * 4 + k;
            const int64_t pos = static_cast<int64_t>(vg) * 32 + (tid & 31);
            if (pos < p.v) cid = p.vocab_order ? p.vocab_order[pos] : static_cast<int>(pos);
          }
          sCellCid[tid] = cid;
        }
      } else {
        if (tid < 128) {
          const int k = li + (tid >> 5);
          int64_t i = p.b;
          if (k < list_n) i = static_cast<int64_t>(use_list ? sList[k] : seg + k) * 32 + (tid & 31);
          load_row_meta(p, i, tid, meta);
        }
      }
      if (tid == 0) sMisc[1] = 0;
      __syncthreads();
      const int* other_ids = IS_DE ? sCellCid : meta.row;
      // Waves and entries: with 3 or 4 entries in the trip wave w recomputes entry w over all of D; with
      // 2 (1) entries, two (four) waves share an entry, each over a half (quarter) of every stage, and the
      // first of them -- the entry's owner -- sums the partial logits and goes on alone.
      const int nent = min(4, list_n - li);
      const int kparts = (nent == 1) ? 4 : ((nent == 2) ? 2 : 1);
      const int ew = wave / kparts;
      const int kpart = wave - ew * kparts;
      const bool owner = (kpart == 0);
      const int entry = li + ew;
      const bool have_entry = entry < list_n;
      const int entry_id = have_entry ? (use_list ? sList[entry] : (IS_DE ? seg * 4 + entry : seg + entry)) : -1;

      // other-side load pointers of this trip (8 per wave and stage)
      const uint16_t* other_ptr[8];
      uint32_t other_live = 0u;  // bit q: load q fetches a real row (advances with the stage)
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const int id = other_ids[4 * (q * 4 + wave) + (lane >> 4)];
        other_ptr[q] = (id < 0) ? zero_chunk : other_base + static_cast<int64_t>(id) * other_sr + lane_chunk;
        other_live |= (id < 0 ? 0u : 1u) << q;
      }
      // Entries are packed at the front of a trip; the rows of absent ones are not fetched (loads
      // 2 e and 2 e + 1 of a wave belong to entry e), so a short trip moves proportionally less data.
      // A short trip has small stages, so more of them fit the ring and more loads are in flight: a
      // stage holds the rows of the present entries followed by the own rows.
      // (The logit phase below has its own compile-time geometry: slots of entries + own rows.  The product phase
      // fetches no own rows, so its slots hold the entries' rows alone and more of them fit the ring: 3 / 5 / 7 / 7
      // slots for 4 / 3 / 2 / 1 entries, light 3 / 6 for 2 / 1 -- 7 at most, the waits below know no deeper ring.)
      const int slot_bytes = 32 * nent * kFRowBytes;
      const int ring = min(7, Lds::kRing / slot_bytes);
      const int ahead = ring - 1;                              // stages in flight
      // product phase: load q of this wave (rows of entry q / 2) for the stage that starts at column col0
      auto issue_load = [&](int q, int col0, int slot, uint32_t entries) {
        if ((entries >> (q >> 1)) & 1u)
          lds_dma16(other_ptr[q] + (((other_live >> q) & 1u) ? col0 : 0), lds_base + slot * slot_bytes + (q * 4 + wave) * 1024);
      };
      auto issue_stage = [&](int col0, int slot, uint32_t entries) {
#pragma unroll
        for (int q = 0; q < 8; ++q) issue_load(q, col0, slot, entries);
      };

      // ---- logits^T of (entry of this wave) x (own rows): 2 nent + 2 loads per wave and stage -----------
      // One wave per SIMD issues every instruction of this loop by itself, so the loop is written once per
      // number of entries: ring geometry, wait counts and which loads exist are then compile-time facts and
      // the body is straight-line code.
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; ++r) s[r] = 0.0f;
      auto logits_of_trip = [&](auto nent_tag) {
        constexpr int NENT = decltype(nent_tag)::value;
        constexpr int KPARTS = (NENT == 1) ? 4 : ((NENT == 2) ? 2 : 1);
        constexpr int NKK = 8 / KPARTS;
        constexpr int OWN_OFF = 32 * NENT * kFRowBytes;
        constexpr int SLOT = OWN_OFF + kFOwnBytes;
        constexpr int RING = Lds::kRing / SLOT;
        constexpr int AHEAD = RING - 1;
        constexpr int PER_STAGE = 2 * NENT + 2;
        auto issue = [&](auto q_tag, int col0, unsigned base) {
          constexpr int Q = decltype(q_tag)::value;
          if constexpr (Q < 2 * NENT) {
            lds_dma16(other_ptr[Q] + (((other_live >> Q) & 1u) ? col0 : 0), base + (Q * 4 + wave) * 1024);
          } else if constexpr (Q >= 8) {
            lds_dma16(own_ptr[Q - 8] + (own_step[Q - 8] ? col0 : 0), base + OWN_OFF + ((Q - 8) * 4 + wave) * 1024);
          }
        };
        // the MFMAs of stage `slot`; with ISSUE the loads of column block next_col go out among them
        auto step = [&](auto issue_tag, int slot, int next_col, int next_slot) {
          constexpr bool ISSUE = decltype(issue_tag)::value;
          const unsigned char* so = smem + slot * SLOT;
          const unsigned char* sw = so + OWN_OFF;
          const unsigned nbase = lds_base + next_slot * SLOT;
          // All fragment reads of a half stage go out first, then loads (their issue is what takes longest in a
          // step: the reads land meanwhile) with the MFMAs in between.
          typename Elem<T>::vec8 fo[4], fw[4];
          auto read_half = [&](int j0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if (j0 + j < NKK) {
                const int kk = kpart * NKK + j0 + j;
                fo[j] = fstage_frag<T>(so, ew * 32 + l32, kk * 2 + half);
                fw[j] = fstage_frag<T>(sw, l32, kk * 2 + half);
              }
            }
          };
          auto mfma_of = [&](int j) {
            if (IS_DE) Elem<T>::mfma_vgpr(fo[j], fw[j], s);
            else Elem<T>::mfma_vgpr(fw[j], fo[j], s);
          };
          read_half(0);
          if constexpr (ISSUE) {
            issue(std::integral_constant<int, 0>{}, next_col, nbase);
            issue(std::integral_constant<int, 1>{}, next_col, nbase);
          }
          static_for<4>([&](auto j) {
            if constexpr (j.value < NKK) mfma_of(j.value);
            if constexpr (ISSUE) issue(std::integral_constant<int, 2 + j.value>{}, next_col, nbase);
          });
          if constexpr (NKK == 8) read_half(4);
          if constexpr (ISSUE) {
            issue(std::integral_constant<int, 6>{}, next_col, nbase);
            issue(std::integral_constant<int, 7>{}, next_col, nbase);
          }
          static_for<4>([&](auto j) {
            if constexpr (NKK == 8) mfma_of(j.value);
            if constexpr (ISSUE && j.value < 2) issue(std::integral_constant<int, 8 + j.value>{}, next_col, nbase);
          });
        };

        const int npre = min(AHEAD, nstages);
#pragma unroll 1
        for (int j = 0; j < npre; ++j)
          static_for<10>([&](auto q) { issue(q, j * kFCols, lds_base + j * SLOT); });
        int slot = 0;  // st % RING
        const int nsteady = nstages - npre;  // steps that still have a stage to start
#pragma unroll 1
        for (int st = 0; st < nsteady; ++st) {
          wait_vmcnt<(AHEAD - 1) * PER_STAGE>();  // all but the newest stages have landed
          __syncthreads();                          // ... for every wave; stage st - 1 is consumed
          const int next_slot = (slot == 0) ? RING - 1 : slot - 1;
          step(std::true_type{}, slot, (st + AHEAD) * kFCols, next_slot);
          slot = (slot + 1 == RING) ? 0 : slot + 1;
        }
#pragma unroll 1
        for (int st = nsteady; st < nstages; ++st) {
          wait_vmcnt_upto((nstages - 1 - st) * PER_STAGE);
          __syncthreads();
          step(std::false_type{}, slot, 0, 0);
          slot = (slot + 1 == RING) ? 0 : slot + 1;
        }
      };
      if (nent >= 3) {
        if constexpr (!LIGHT) logits_of_trip(std::integral_constant<int, 4>{});
      } else if (nent == 2) {
        logits_of_trip(std::integral_constant<int, 2>{});
      } else {
        logits_of_trip(std::integral_constant<int, 1>{});
      }
      mfma_drain(s);
      __syncthreads();  // every load has landed and every stage is consumed
      if (kparts > 1) {  // partial logits -> the owner, through the idle ring, in a fixed order
        float* sRed = reinterpret_cast<float*>(smem);
        if (!owner) {
#pragma unroll
          for (int r = 0; r < 16; ++r) sRed[(wave * 16 + r) * 64 + lane] = s[r];
        }
        __syncthreads();
        if (owner) {
          for (int q = 1; q < kparts; ++q) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] += sRed[((wave + q) * 16 + r) * 64 + lane];
          }
        }
        __syncthreads();  // before the product phase refills the ring
      }

      // ---- dz of the owner's 32 x 32 block (lane = token row, registers = classes) ----------------------------
      if (owner) {
        const int mrow = IS_DE ? l32 : ew * 32 + l32;
        const int* cid32 = IS_DE ? sCellCid + ew * 32 : sOwnCid;
        const bool big = block_epilogue<T>(p, s, cid32, half, meta.lse2[mrow], meta.g[mrow], meta.h[mrow], meta.tgt[mrow]);
        bool use = have_entry;
        if (IS_DE) {
          const bool survives = (p.filter_eps < 0.0f) || (__ballot(big) != 0ull);
          const bool live = have_entry && (static_cast<int64_t>(entry_id) * 32 < p.v);
          use = live && (survives || !p.filter_e);
          if (lane == 0 && live && survives) atomicOr(&sBits[entry_id >> 5], 1u << (entry_id & 31));
          if (lane == 0 && live) n_recomputed += 1;
        }
        if (use) {
          if (IS_DE) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
              const int k = ew * 32 + 8 * r4 + 4 * half;
              uint2 pk;
              pk.x = Elem<T>::pack2(s[r4 * 4 + 0], s[r4 * 4 + 1]);
              pk.y = Elem<T>::pack2(s[r4 * 4 + 2], s[r4 * 4 + 3]);
              *reinterpret_cast<uint2*>(sDz + l32 * 256 + ((((k >> 3) ^ (l32 & 7)) << 4) | ((k & 7) << 1))) = pk;
            }
          } else {
            const int k = ew * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int cls = 8 * (r >> 2) + 4 * half + (r & 3);
              *reinterpret_cast<uint16_t*>(sDz + cls * 256 + ((((k >> 3) ^ (cls & 7)) << 4) | ((k & 7) << 1))) =
                  Elem<T>::from_float(s[r]);
              if (p.d_bias != nullptr) {
                float colsum = s[r];
#pragma unroll
                for (int off = 16; off >= 1; off >>= 1) colsum += __shfl_xor(colsum, off, 64);
                if (l32 == 0) sDb[ew * 32 + cls] += colsum;
              }
            }
          }
          if (lane == 0) atomicOr(&sMisc[1], 1 << ew);
        }
      }
      __syncthreads();
      const uint32_t mask = static_cast<uint32_t>(sMisc[1]);
      const bool product = write_out && (mask != 0u);
      if (mask != 0u) {
        touched = true;
        if (tid == 0) n_product += __popc(mask);
      }

      // ---- own_grad^T (D x 32) += Other_cell^T . dz, 128 columns of D per stage --------------------------------------
      typename Elem<T>::vec8 bz[8];
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        const uint4 v = *reinterpret_cast<const uint4*>(sDz + l32 * 256 + (((kk * 2 + half) ^ (l32 & 7)) << 4));
        bz[kk] = __builtin_bit_cast(typename Elem<T>::vec8, v);
      }
      if (product) {
        // Only the entries that are used are fetched again: the others would be read for nothing.
        const int nused = __popc(mask);
        const int npre = min(ahead, nchunks);
#pragma unroll 1
        for (int j = 0; j < npre; ++j) issue_stage(d_begin + j * kFCols, j, mask);
        int pslot = 0;  // ci % ring
        auto product_chunk = [&](int ci, f32x16& accum, auto in_agpr) {
          // The stages after ci may be in flight -- and, in the light variant, the stores of the chunks whose loads
          // were issued after those of ci (memory operations of a wave complete in issue order and share one counter;
          // a wait that forgot the stores would wait for the newest loads and for the stores' acknowledgements).
          if constexpr (LIGHT) wait_vmcnt_upto_wide(min(ahead - 1, nchunks - 1 - ci) * 2 * nused + kLightStores * min(ahead, ci));
          else wait_vmcnt_upto(min(ahead - 1, nchunks - 1 - ci) * 2 * nused);
          __syncthreads();
          const unsigned char* so = smem + pslot * slot_bytes;
          const int next_col = d_begin + (ci + ahead) * kFCols;
          const uint32_t next_mask = (ci + ahead < nchunks) ? mask : 0u;  // nothing is fetched past the slice
          const int next_slot = (pslot == 0) ? ring - 1 : pslot - 1;
          pslot = (pslot + 1 == ring) ? 0 : pslot + 1;
          // as in the logit phase: reads, then loads with the MFMAs in between
          typename Elem<T>::vec8 a[4];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if ((mask >> ((4 * h + j) >> 1)) & 1u) a[j] = fstage_frag_transposed<T>(so, (4 * h + j) * 16, wave * 32, lane);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int kk = 4 * h + j;
              issue_load(kk, next_col, next_slot, next_mask);
              if ((mask >> (kk >> 1)) & 1u) {
                if constexpr (decltype(in_agpr)::value) Elem<T>::mfma_agpr(a[j], bz[kk], accum);
                else Elem<T>::mfma_vgpr(a[j], bz[kk], accum);
              }
            }
          }
        };
        if constexpr (LIGHT) {
          // one chunk at a time: formed, written straight from the registers (8 bytes per lane and row piece), gone
#pragma unroll 1
          for (int ci = 0; ci < nchunks; ++ci) {
            product_chunk(ci, acc[0], std::false_type{});
            mfma_drain(acc[0]);
            store_chunk_direct(ci, acc[0]);
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[0][r] = 0.0f;
          }
        } else {
#pragma unroll
          for (int ci = 0; ci < kFMaxChunks; ++ci) {
            if (ci < nchunks) {
              if (ci < 16) product_chunk(ci, acc[ci], std::true_type{});  // 16 chunks fill the 256 AGPRs
              else product_chunk(ci, acc[ci], std::false_type{});
            }
          }
        }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // drain before the ring is refilled
      __syncthreads();
    }
    carry = keep_rest ? list_n - run_n : 0;
    if (tid < carry) {  // wave 0, which also builds the next list: LDS operations of one wave stay in order
      const int rest = sList[run_n + tid];
      sList[tid] = rest;
    }
  }

  mfma_drain_all();  // the last product MFMAs, before anything else reads the accumulators
  const bool out_fp32 = IS_DE ? (p.de_fp32 != 0) : (p.dc_fp32 != 0);
  if constexpr (LIGHT) {
    if (write_out && !touched) {
      // Nothing survived for this class group: its rows are zeros, written as whole 16-byte pieces, a wave
      // instruction inside one row (the launcher guarantees 16-byte aligned rows and D a multiple of 128).
      const int ppr = (d_end - d_begin) / 8;  // 16-byte pieces per row
      const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
      for (int j = tid; j < 32 * ppr; j += kBwdThreads) {
        const int row = j / ppr;
        const int id = own_ids[row];
        if (id >= 0)
          *reinterpret_cast<uint4*>(static_cast<uint16_t*>(p.d_c) + static_cast<int64_t>(id) * own_sr + d_begin +
                                    (j - row * ppr) * 8) = zero;
      }
    }
  } else if (write_out && (touched || !IS_DE)) {  // dC rows are always written; the launcher guarantees 16-byte aligned rows
    // The accumulators hold the tile transposed (lane = own row, registers = columns): stored as they
    // are, one instruction would touch 32 rows with 16 bytes each.  Four chunks at a time go through
    // LDS instead and leave as whole rows, 16 bytes per lane and 1 KB per row and instruction.
    unsigned char* out_base = static_cast<unsigned char*>(IS_DE ? p.d_e : p.d_c);
    auto store_tile = [&](auto fp32_tag) {
      constexpr bool FP32 = decltype(fp32_tag)::value;
      constexpr int es = FP32 ? 4 : 2;
      constexpr int pitch = 4 * kFCols * es + 16;  // the odd 16 bytes spread the rows over the banks
#pragma unroll
      for (int g = 0; g < (kFMaxChunks + 3) / 4; ++g) {
        if (g * 4 < nchunks) {
          __syncthreads();  // the ring is idle / the previous group has been read
#pragma unroll
          for (int cj = 0; cj < 4; ++cj) {
            constexpr int kLast = kFMaxChunks - 1;
            const int ci = g * 4 + cj;
            if (ci <= kLast && ci < nchunks) {
              // an accumulator that was pinned to the AGPRs stays there until this very point: otherwise
              // the compiler moves all of them to ordinary registers (and on to scratch) before the loop
              if (ci < 16) asm volatile("" : "+a"(acc[ci <= kLast ? ci : kLast]));
              const f32x16& a = acc[ci <= kLast ? ci : kLast];
#pragma unroll
              for (int r4 = 0; r4 < 4; ++r4) {
                unsigned char* dst = smem + l32 * pitch + (cj * kFCols + wave * 32 + 8 * r4 + 4 * half) * es;
                if (FP32) {
                  *reinterpret_cast<float4*>(dst) = make_float4(a[r4 * 4 + 0], a[r4 * 4 + 1], a[r4 * 4 + 2], a[r4 * 4 + 3]);
                } else {
                  uint2 pk;
                  pk.x = Elem<T>::pack2(a[r4 * 4 + 0], a[r4 * 4 + 1]);
                  pk.y = Elem<T>::pack2(a[r4 * 4 + 2], a[r4 * 4 + 3]);
                  *reinterpret_cast<uint2*>(dst) = pk;
                }
              }
            }
          }
          __syncthreads();
          // 16-byte pieces per row: a multiple of 16, so one wave instruction stays inside one row and the
          // 32 rows make at least two pieces per thread; two are read before either is stored.
          const int ppr = min(4, nchunks - g * 4) * kFCols * es / 16;
          for (int j = tid; j < 32 * ppr; j += 2 * kBwdThreads) {
            const int ja = j, jb = j + kBwdThreads;
            const int rowa = ja / ppr, rowb = jb / ppr;
            const int pca = ja - rowa * ppr, pcb = jb - rowb * ppr;
            const int ida = own_ids[rowa], idb = own_ids[rowb];
            const uint4 va = *reinterpret_cast<const uint4*>(smem + rowa * pitch + pca * 16);
            const uint4 vb = *reinterpret_cast<const uint4*>(smem + rowb * pitch + pcb * 16);
            const int64_t col_bytes = static_cast<int64_t>(d_begin + g * 4 * kFCols) * es;
            if (ida >= 0)
              *reinterpret_cast<uint4*>(out_base + static_cast<int64_t>(ida) * own_sr * es + col_bytes + pca * 16) = va;
            if (idb >= 0)
              *reinterpret_cast<uint4*>(out_base + static_cast<int64_t>(idb) * own_sr * es + col_bytes + pcb * 16) = vb;
          }
        }
      }
    };
    if (out_fp32) store_tile(std::true_type{});
    else store_tile(std::false_type{});
  }
  if (slice == 0) {
    if (IS_DE) {
      if (p.kept_bits != nullptr)
        for (int w = tid; w < p.bit_words; w += kBwdThreads)
          p.kept_bits[static_cast<int64_t>(own) * p.bit_words + w] = sBits[w];
      if (p.counters != nullptr) {
        if (lane == 0 && n_recomputed) atomicAdd(p.counters + 1, n_recomputed);
        if (tid == 0 && n_product) atomicAdd(p.counters + 2, n_product);
        if (tid == 0 && blockIdx.x == 0)
          atomicAdd(p.counters + 0, static_cast<unsigned long long>(p.ntg) * static_cast<unsigned long long>(p.nvg));
      }
    } else {
      if (p.d_bias != nullptr && touched && tid < 32 && sOwnCid[tid] >= 0)
        p.d_bias[sOwnCid[tid]] = (sDb[tid] + sDb[32 + tid]) + (sDb[64 + tid] + sDb[96 + tid]);
      if (p.counters != nullptr && tid == 0 && n_product) atomicAdd(p.counters + 3, n_product);
    }
  }
}

// Number of cells of the forward statistic (32 rows x 32 classes) whose bound exp(max logit - min lse of the 32
// rows) reaches eps: the cells the ownership kernels have to recompute.  One workgroup per row group.
__global__ __launch_bounds__(256) void flagged_cells_kernel(const float* tile_max, const float* lse, int64_t b, int stat_cols,
                                                            float log_eps, unsigned long long* count) {
  __shared__ float s_min;
  __shared__ unsigned int s_part[4];
  const int tg = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (wave == 0) {
    const int64_t i = static_cast<int64_t>(tg) * 32 + lane;
    const float mn = wave_min((lane < 32 && i < b) ? lse[i] : INFINITY);
    if (lane == 0) s_min = mn;
  }
  __syncthreads();
  const float min_lse = s_min;
  const float* row = tile_max + static_cast<int64_t>(tg) * stat_cols;
  unsigned int n = 0;
  for (int j = threadIdx.x; j < stat_cols; j += 256) n += (row[j] - min_lse >= log_eps) ? 1u : 0u;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) n += __shfl_xor(n, off, 64);
  if (lane == 0) s_part[wave] = n;
  __syncthreads();
  if (threadIdx.x == 0) atomicAdd(count, static_cast<unsigned long long>(s_part[0] + s_part[1] + s_part[2] + s_part[3]));
}

}  // namespace cce

using namespace cce;

extern "C" int cce_count_flagged_cells(const float* tile_max, const float* lse, int64_t b, int64_t v, float filter_eps,
                                       uint64_t* count, void* stream_) {
  if (b < 0 || v <= 0 || !(filter_eps > 0.0f)) return CCE_ERR_INVALID_ARGUMENT;
  if (b == 0) return CCE_OK;
  if (tile_max == nullptr || lse == nullptr || count == nullptr) return CCE_ERR_INVALID_ARGUMENT;
  const int64_t ntg = (b + CCE_STAT_ROWS - 1) / CCE_STAT_ROWS;
  if (ntg >= (int64_t(1) << 31) || v >= (int64_t(1) << 31) - 512) return CCE_ERR_INVALID_ARGUMENT;
  const int stat_cols = static_cast<int>((v + CCE_STAT_COLS - 1) / CCE_STAT_COLS);
  hipLaunchKernelGGL(flagged_cells_kernel, dim3(static_cast<unsigned>(ntg)), dim3(256), 0, static_cast<hipStream_t>(stream_),
                     tile_max, lse, b, stat_cols, logf(filter_eps) - 0.01f,
                     reinterpret_cast<unsigned long long*>(count));
  return status_from_hip(hipGetLastError());
}

static int64_t bit_words_for(int64_t v) { return ((v + 31) / 32 + 31) / 32; }

// survivor bits, then the list of class groups for the full dC pass (a count and up to one id per group)
static int64_t kept_bits_bytes(int64_t b, int64_t v) { return ((b + 31) / 32) * bit_words_for(v) * 4; }

extern "C" int64_t cce_backward_workspace_bytes(int64_t b, int64_t v, int64_t d) {
  (void)d;
  if (b <= 0 || v <= 0) return 0;
  return kept_bits_bytes(b, v) + (1 + (v + 31) / 32) * 4;
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
  if (bit_words_for(v) > kMaxBitWords) return CCE_ERR_INVALID_ARGUMENT;

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
  p.light_on = 0;
  p.heavy_list = nullptr;

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
    p.heavy_list = reinterpret_cast<int*>(static_cast<unsigned char*>(workspace) + kept_bits_bytes(b, v));
  }
  // Cells may be skipped unseen only if a filtered sub-tile feeds nothing this pass produces.
  p.shortcut = (tile_max != nullptr && vocab_order == nullptr && filtering && filter_eps > 0.0f &&
                (d_e == nullptr || p.filter_e)) ? 1 : 0;

  const bool aligned = aligned16(e) && aligned16(c) && (d % 8 == 0) && (stride_e % 8 == 0) &&
                       (stride_cv % 8 == 0) && (stride_cd == 1);
  // The fast kernels want whole 128-column stages, also inside every slice of D.
  // ... and they store whole 16-byte pieces of the output rows.
  const bool fast = aligned && (d % kFCols == 0) && (d_e == nullptr || p.vec_e) && (d_c == nullptr || p.vec_c);
  hipError_t err;
#define CCE_LAUNCH(KERN, LDS, GRID)                                                                 \
  do {                                                                                              \
    auto kern = KERN;                                                                               \
    static LdsLimitOnce lds_limit;                                                            \
    err = lds_limit.set(kern, LDS);                                        \
    if (err != hipSuccess) return status_from_hip(err);                                             \
    hipLaunchKernelGGL(kern, dim3(GRID), dim3(kBwdThreads), LDS, stream, p);                        \
  } while (0)
#define CCE_LAUNCH_OWNER(IS_DE_, GRID)                                                              \
  do {                                                                                              \
    if (dtype == CCE_DTYPE_BF16) {                                                                  \
      if (fast) CCE_LAUNCH((bwd_owner_fast_kernel<BF16, IS_DE_>), kFLdsBytes, GRID);                \
      else if (aligned) CCE_LAUNCH((bwd_owner_kernel<BF16, true, IS_DE_>), kBwdLdsBytes, GRID);     \
      else CCE_LAUNCH((bwd_owner_kernel<BF16, false, IS_DE_>), kBwdLdsBytes, GRID);                 \
    } else {                                                                                        \
      if (fast) CCE_LAUNCH((bwd_owner_fast_kernel<F16, IS_DE_>), kFLdsBytes, GRID);                 \
      else if (aligned) CCE_LAUNCH((bwd_owner_kernel<F16, true, IS_DE_>), kBwdLdsBytes, GRID);      \
      else CCE_LAUNCH((bwd_owner_kernel<F16, false, IS_DE_>), kBwdLdsBytes, GRID);                  \
    }                                                                                               \
  } while (0)
  const int full_slices = p.nslices;
  if (need_de_pass) {
    p.nslices = (d_e != nullptr) ? full_slices : 1;
    const unsigned grid = static_cast<unsigned>(p.ntg) * static_cast<unsigned>(p.nslices);
    CCE_LAUNCH_OWNER(true, grid);
    err = hipGetLastError();
    if (err != hipSuccess) return status_from_hip(err);
  }
  if (need_dc_pass) {
    // Class groups with at most two surviving entries (most of them when rows are few against the classes) go to a
    // light variant of the same kernel that holds no gradient in registers and shares a compute unit two by two:
    // what such a group costs is latency, not work.  It wants a filtered 16-bit dC and one list segment; it
    // covers all of D itself.  The full variant then skips those groups.
    const bool light = fast && d_c != nullptr && !d_c_is_fp32 && p.filter_c && p.ntg <= kFListCap;
    if (light) {
      BwdParams q = p;
      q.nslices = 1;
      q.dslice = static_cast<int>(d);
      const unsigned grid = static_cast<unsigned>(q.nvg);
      if (dtype == CCE_DTYPE_BF16) {
        auto kern = bwd_owner_fast_kernel<BF16, false, true>;
        static LdsLimitOnce lds_limit;
        err = lds_limit.set(kern, kFLightLdsBytes);
        if (err != hipSuccess) return status_from_hip(err);
        hipLaunchKernelGGL(kern, dim3(grid), dim3(kBwdThreads), kFLightLdsBytes, stream, q);
      } else {
        auto kern = bwd_owner_fast_kernel<F16, false, true>;
        static LdsLimitOnce lds_limit;
        err = lds_limit.set(kern, kFLightLdsBytes);
        if (err != hipSuccess) return status_from_hip(err);
        hipLaunchKernelGGL(kern, dim3(grid), dim3(kBwdThreads), kFLightLdsBytes, stream, q);
      }
      err = hipGetLastError();
      if (err != hipSuccess) return status_from_hip(err);
      p.light_on = 1;
    }
    p.nslices = (d_c != nullptr) ? full_slices : 1;
    const unsigned grid = static_cast<unsigned>(p.nvg) * static_cast<unsigned>(p.nslices);
    CCE_LAUNCH_OWNER(false, grid);
  }
#undef CCE_LAUNCH_OWNER
#undef CCE_LAUNCH
  return status_from_hip(hipGetLastError());
}
