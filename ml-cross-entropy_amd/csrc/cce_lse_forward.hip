// cce_lse_forward: fused (E . C^T) -> soft-cap -> online log-sum-exp for gfx950.
//
// Work decomposition.  The (row-block, vocabulary) plane is cut into items: one item is a block
// of 256 valid rows times a contiguous span of 256-wide vocabulary tiles.  A workgroup (8 waves,
// 2 x 4, each wave 128 classes x 64 rows of accumulators) owns one item, walks its span tile by
// tile and keeps, per row, a running (max, sum-exp) pair in registers in the log2 domain.  At the
// end the pairs of the two lane halves and of the two wave rows are merged and written as one
// partial per (span, row); a second tiny kernel merges the spans.  No lock and no atomic is
// needed and the result is deterministic.
//
// Workgroup ids are dealt round-robin to the 8 XCDs by the hardware, so the id is first turned
// into (xcd, slot) and items are numbered so that one XCD works on neighbouring spans of the
// same few row blocks: its L2 then serves each E block to several workgroups and each C tile to
// several row blocks.
#include <atomic>

#include "cce_common.h"

namespace cce {

struct LseFwdParams {
  const uint16_t* e;
  const uint16_t* c;
  const uint16_t* bias;
  const int32_t* valids;
  float* logit_avg;
  float* tile_max;
  float2* partial;  // [nsplit][b] (max2, sum)
  int64_t b, v, d, n_rows;
  int64_t stride_e, stride_cv, stride_cd;
  int nrb, nvt, nsplit, nitems, items_per_xcd;
  int stat_cols;
  Softcap sc;
  float avg_scale;  // ln 2 / b: turns a column sum in log2 units into its share of logit_avg
  float cap_inv;    // 1 / (-2 cap log2(e)) (soft-capping on), for the fixed-reference epilogue
};

// 8 waves (two per SIMD, so that one wave's LDS and global traffic issues in the shadow of the
// other's MFMAs), 2 x 4: each wave owns 128 classes x 64 rows of the 256 x 256 tile.
constexpr int kFwdWV = 4, kFwdWT = 2, kFwdNWV = 2, kFwdNWT = 4;
constexpr int kFwdThreads = 64 * kFwdNWV * kFwdNWT;
constexpr int kFwdTile = 256;
static_assert(32 * kFwdWV * kFwdNWV == kFwdTile && 32 * kFwdWT * kFwdNWT == kFwdTile, "tile is 256 x 256");
static_assert(CCE_STAT_COLS == 32 && CCE_STAT_ROWS == 32, "one statistic cell per 32 x 32 accumulator block");

constexpr int kFwdBiasBytes = 2 * 256 * 4;  // two tiles' worth of per-class addends (double-buffered)

// Soft-capped logits (log2 domain) of one 32-row column block of a wave: 4 class blocks x 16 registers.
// GENERAL adds a per-class addend staged in LDS: the bias (or 0), or -inf for a class past the end of
// the vocabulary, which is masked AFTER soft-capping (soft-capping -inf would give -softcap, not -inf).
// The plain variant is straight-line code with no loads.
template <bool GENERAL, bool CAP>
__device__ __forceinline__ float column_block_logits_impl(const Softcap& sc, const f32x16 (&acc)[kFwdWV][kFwdWT], int ti,
                                                          const float* addend, int half, float (&s2)[kFwdWV][16],
                                                          float (&bm)[kFwdWV]) {
  float tm = -INFINITY;
#pragma unroll
  for (int vi = 0; vi < kFwdWV; ++vi) {
    bm[vi] = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float x = acc[vi][ti][r];
      bool dead = false;
      if (GENERAL) {
        const float add = addend[vi * 32 + 8 * (r >> 2) + 4 * half + (r & 3)];
        dead = (add == -INFINITY);
        x = dead ? 0.0f : x + add;
      }
      float y;
      if (CAP) {
        // cap * log2(e) * tanh(x / cap), tanh(u) = 1 - 2 / (1 + exp(2 u))
        const float t = __builtin_amdgcn_exp2f(x * sc.in_scale);
        const float w = __builtin_amdgcn_rcpf(1.0f + t);
        y = fmaf(w, -2.0f * sc.out_scale, sc.out_scale);
      } else {
        y = x * kLog2e;
      }
      s2[vi][r] = dead ? -INFINITY : y;
      bm[vi] = fmaxf(bm[vi], s2[vi][r]);
    }
    tm = fmaxf(tm, bm[vi]);
  }
  return tm;
}

// One uniform branch per column block: each arm is straight-line code over all 64 values, so the
// independent exp2 / rcp chains of different values overlap.
template <bool GENERAL>
__device__ __forceinline__ float column_block_logits(const Softcap& sc, const f32x16 (&acc)[kFwdWV][kFwdWT], int ti,
                                                     const float* addend, int half, float (&s2)[kFwdWV][16],
                                                     float (&bm)[kFwdWV]) {
  if (sc.on) return column_block_logits_impl<GENERAL, true>(sc, acc, ti, addend, half, s2, bm);
  return column_block_logits_impl<GENERAL, false>(sc, acc, ti, addend, half, s2, bm);
}

// Kernel variants:
//   FAST     rows 16-byte aligned, unit column stride, D % 64 == 0: direct-to-LDS pipelined main loop
//   ALIGNED  (generic main loop only) 16-byte vector loads are legal
//   GENERAL  a bias is present or V is not a multiple of the tile: per-class addend / mask from LDS
//   WANT_LA  also accumulate the column average of the logits (needs GENERAL)
template <typename T, bool FAST, bool ALIGNED, bool GENERAL, bool WANT_LA>
__global__ __launch_bounds__(kFwdThreads, 1) void lse_forward_kernel(LseFwdParams p) {
  using Tile = LogitTile<T, kFwdWV, kFwdWT, kFwdNWV, kFwdNWT, ALIGNED>;
  using Fast = DmaLogitTile<T, kFwdWV, kFwdWT, kFwdNWV, kFwdNWT>;
  static_assert(!WANT_LA || GENERAL, "the column average uses the general epilogue");
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_addend = reinterpret_cast<float*>(smem + Tile::LDS_BYTES);  // [2][256]

  // XCD-aware item id: workgroup ids that land on one XCD get consecutive items.
  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  if (slot >= p.items_per_xcd) return;
  const int item = xcd * p.items_per_xcd + slot;
  if (item >= p.nitems) return;
  const int rb = item / p.nsplit;
  const int split = item % p.nsplit;
  const int vt_begin = static_cast<int>((static_cast<int64_t>(p.nvt) * split) / p.nsplit);
  const int vt_end = static_cast<int>((static_cast<int64_t>(p.nvt) * (split + 1)) / p.nsplit);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wv = wave / kFwdNWT;
  const int wt = wave % kFwdNWT;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int64_t t0 = static_cast<int64_t>(rb) * Tile::TILE_T;

  typename Tile::CLoader cl;
  typename Tile::ELoader el;
  const uint16_t* fptr[Fast::NQ];  // FAST: per-lane source of each direct-to-LDS load
  if (FAST) {
#pragma unroll
    for (int q = Fast::NQC; q < Fast::NQ; ++q) {
      int64_t i = t0 + Fast::row_of(q, wave, lane);
      i = (i < p.b) ? i : p.b - 1;  // rows past the end repeat the last one; their results are dropped
      const int64_t row = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
      fptr[q] = p.e + row * p.stride_e + Fast::chunk_elems(wave, lane);
    }
  } else {
#pragma unroll
    for (int q = 0; q < Tile::ELoader::NQ; ++q) {
      const int64_t i = t0 + (tid >> 3) + q * Tile::ELoader::ROWSTEP;
      const uint16_t* ptr = nullptr;
      if (i < p.b) {
        const int64_t row = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
        ptr = p.e + row * p.stride_e;
      }
      el.ptr[q] = ptr;
    }
  }

  float m2[kFwdWT], sum[kFwdWT];
#pragma unroll
  for (int ti = 0; ti < kFwdWT; ++ti) {
    m2[ti] = -INFINITY;
    sum[ti] = 0.0f;
  }

  auto set_class_pointers = [&](int64_t v0) {
#pragma unroll
    for (int q = 0; q < Fast::NQC; ++q) {
      int64_t vr = v0 + Fast::row_of(q, wave, lane);
      vr = (vr < p.v) ? vr : p.v - 1;  // classes past the end repeat the last one; masked in the epilogue
      fptr[q] = p.c + vr * p.stride_cv + Fast::chunk_elems(wave, lane);
    }
  };

  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int64_t v0 = static_cast<int64_t>(vt) * Tile::TILE_V;
    float* addend = s_addend + (vt & 1) * kFwdTile;
    if (GENERAL) {
      // Written before the main loop, whose barriers publish it; the other buffer may still be read
      // by a wave that is finishing the previous tile.
      if (tid < kFwdTile) {
        const int64_t vg = v0 + tid;
        float a = -INFINITY;
        if (vg < p.v) a = (p.bias != nullptr) ? Elem<T>::to_float(p.bias[vg]) : 0.0f;
        addend[tid] = a;
      }
    }
    f32x16 acc[kFwdWV][kFwdWT];
    if (FAST) {
      if (vt == vt_begin) {
        set_class_pointers(v0);
        Fast::prefetch(fptr, smem, static_cast<int>(p.d));
      }
      Fast::run(acc, fptr, smem, static_cast<int>(p.d));
      if (vt + 1 < vt_end) {
        // the ring is idle during the epilogue: start on the next tile now
        set_class_pointers(v0 + Tile::TILE_V);
        Fast::prefetch(fptr, smem, static_cast<int>(p.d));
      }
    } else {
#pragma unroll
      for (int q = 0; q < Tile::CLoader::NQ; ++q) {
        const int64_t vr = v0 + (tid >> 3) + q * Tile::CLoader::ROWSTEP;
        cl.ptr[q] = (vr < p.v) ? p.c + vr * p.stride_cv : nullptr;
      }
      Tile::run(acc, cl, el, smem, static_cast<int>(p.d), p.stride_cd);
    }

    // ---- epilogue: (bias, mask,) soft-cap, online max / sum-exp ---------------------------------
    // One 32-row column block at a time, so that only 64 soft-capped logits are live at once.
    const int64_t vw0 = v0 + wv * (32 * kFwdWV);  // first class of this wave
    const float* wave_addend = addend + wv * (32 * kFwdWV);
#pragma unroll
    for (int ti = 0; ti < kFwdWT; ++ti) {
      __builtin_amdgcn_sched_barrier(0);  // keep each column block's register use to itself
      float s2[kFwdWV][16];
      float bm[kFwdWV];  // this lane's maximum in each of the four 32-class blocks
      const float tm = column_block_logits<GENERAL>(p.sc, acc, ti, wave_addend, half, s2, bm);
      if (WANT_LA) {
        // Column sums over the 32 rows of this block, in natural-log units, added to the running average right
        // away: nothing is carried from one column block to the next, so asking for the average costs the
        // direct-to-LDS kernel no registers beyond these temporaries.
        const float ok = (t0 + wt * (32 * kFwdWT) + ti * 32 + l32 < p.b) ? 1.0f : 0.0f;
        const float inv_b = kLn2 / static_cast<float>(p.b);
        float* avg = p.logit_avg + vw0 + 4 * half;                 // this lane half's first class of the wave
        const int left = static_cast<int>(min(p.v - vw0, static_cast<int64_t>(32 * kFwdWV))) - 4 * half;
#pragma unroll
        for (int vi = 0; vi < kFwdWV; ++vi) {
          __builtin_amdgcn_sched_barrier(0);  // one 32-class block at a time
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int cls = vi * 32 + 8 * (r >> 2) + (r & 3);
            float cs = (s2[vi][r] == -INFINITY) ? 0.0f : s2[vi][r] * ok;
#pragma unroll
            for (int off = 16; off >= 1; off >>= 1) cs += __shfl_xor(cs, off, 64);
            if (l32 == 0 && cls < left) unsafeAtomicAdd(avg + cls, cs * inv_b);
          }
        }
      }

      if (p.tile_max != nullptr) {
        // max over the 32 rows x 32 classes of each accumulator block of this (wave, ti)
        const int64_t srow = (t0 + wt * (32 * kFwdWT) + ti * 32) / CCE_STAT_ROWS;
        const int64_t scol = vw0 / CCE_STAT_COLS;
        float cell[kFwdWV];
#pragma unroll
        for (int vi = 0; vi < kFwdWV; ++vi) cell[vi] = wave_max(bm[vi]);
        if (lane < kFwdWV && (t0 + wt * (32 * kFwdWT) + ti * 32) < p.b && vw0 + lane * 32 < p.v) {
          float mine = cell[0];
#pragma unroll
          for (int vi = 1; vi < kFwdWV; ++vi) mine = (lane == vi) ? cell[vi] : mine;
          p.tile_max[srow * p.stat_cols + scol + lane] = mine * kLn2;
        }
      }

      const float mn = fmaxf(m2[ti], tm);
      const float ms = (mn == -INFINITY) ? 0.0f : mn;
      float part = 0.0f;
#pragma unroll
      for (int vi = 0; vi < kFwdWV; ++vi)
#pragma unroll
        for (int r = 0; r < 16; ++r) part += __builtin_amdgcn_exp2f(s2[vi][r] - ms);
      sum[ti] = sum[ti] * __builtin_amdgcn_exp2f(m2[ti] - ms) + part;
      m2[ti] = mn;
    }

  }

  // ---- merge the two lane halves, then the two wave rows, and emit one partial per row -------
  float2* stage = reinterpret_cast<float2*>(smem);  // [NWT][WT][32]
#pragma unroll
  for (int ti = 0; ti < kFwdWT; ++ti) {
    const float om = __shfl_xor(m2[ti], 32, 64);
    const float os = __shfl_xor(sum[ti], 32, 64);
    const float mn = fmaxf(m2[ti], om);
    const float ms = (mn == -INFINITY) ? 0.0f : mn;
    sum[ti] = sum[ti] * __builtin_amdgcn_exp2f(m2[ti] - ms) + os * __builtin_amdgcn_exp2f(om - ms);
    m2[ti] = mn;
  }
  if (wv == 1 && half == 0) {
#pragma unroll
    for (int ti = 0; ti < kFwdWT; ++ti) stage[(wt * kFwdWT + ti) * 32 + l32] = make_float2(m2[ti], sum[ti]);
  }
  __syncthreads();
  if (wv == 0 && half == 0) {
#pragma unroll
    for (int ti = 0; ti < kFwdWT; ++ti) {
      const float2 o = stage[(wt * kFwdWT + ti) * 32 + l32];
      const float mn = fmaxf(m2[ti], o.x);
      const float ms = (mn == -INFINITY) ? 0.0f : mn;
      const float s = sum[ti] * __builtin_amdgcn_exp2f(m2[ti] - ms) + o.y * __builtin_amdgcn_exp2f(o.x - ms);
      const int64_t i = t0 + wt * (32 * kFwdWT) + ti * 32 + l32;
      if (i < p.b) p.partial[static_cast<int64_t>(split) * p.b + i] = make_float2(mn, s);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The direct-to-LDS kernel on 16 x 16 x 32 MFMAs (DmaLogitTile16): same items, tile, ring and partials as
// above; a lane holds, per 16-row block ti of its wave, ONE token row (lane % 16) and the 32 classes
// 16 vi + 4 (lane / 16) + r of the wave's 128.  The epilogue takes two such blocks (32 rows, one row of
// statistic cells) at a time: 64 soft-capped logits live.
// ---------------------------------------------------------------------------------------------
constexpr int kF16WV = 8, kF16WT = 4;  // 16-row blocks per wave: 128 classes x 64 rows
constexpr int kF16RunBytes = kF16WT * kFwdThreads * static_cast<int>(sizeof(float2));  // running (max, sum) pairs
constexpr int kF16ColsumBytes = 2 * kFwdTile * static_cast<int>(sizeof(float));       // column sums (logit_avg only)
static_assert(16 * kF16WV * kFwdNWV == kFwdTile && 16 * kF16WT * kFwdNWT == kFwdTile, "tile is 256 x 256");

// One row block (16 token rows x the wave's 128 classes; 32 values of ONE row per lane) of the epilogue: soft-cap,
// the lane's maximum per 32-class group (for the statistic cells) and the update of the row's running (max, sum-exp).
//
// FIXED: soft-capping with a cap small enough that 2^(-2 cap log2(e)) is a normal float.  Soft-capped logits never
// exceed the cap, so the cap itself is the reference of every row's sum of exponentials -- no running maximum, no
// rescaling, and with w = 1 / (1 + exp(2 x / cap)):  softcap(x) - cap = -2 cap w, so a term of the sum is
// 2^(-2 cap log2(e) w): two instructions fewer per logit than soft-cap, subtract, exponentiate.  The cell maxima are
// taken on the raw logits (soft-capping is monotone) and soft-capped once per cell.  The running pair then holds
// (cap log2(e), sum) and merges with the other spans' pairs like any other.
template <bool GENERAL, bool CAP, bool FIXED, bool WANT_S2>
__device__ __forceinline__ void row_block_impl(const Softcap& sc, float cap_inv, const f32x4 (&acc)[kF16WV][kF16WT], int ti,
                                               const float* addend, int kq, float2& run, float (&bm)[kF16WV / 2],
                                               float (&s2)[kF16WV][4]) {
  float y[kF16WV][4];
  float tm = -INFINITY;
  float part = 0.0f;
#pragma unroll
  for (int vi = 0; vi < kF16WV; ++vi) {
    float gm = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float x = acc[vi][ti][r];
      bool dead = false;
      if (GENERAL) {
        const float add = addend[vi * 16 + 4 * kq + r];
        dead = (add == -INFINITY);
        x = dead ? 0.0f : x + add;
      }
      if (FIXED) {
        // z = -2 cap log2(e) / (1 + t) in one fma and one reciprocal: (1 + t) / k = t / k + 1 / k
        const float t = __builtin_amdgcn_exp2f(x * sc.in_scale);
        const float z = __builtin_amdgcn_rcpf(fmaf(t, cap_inv, cap_inv));
        const float term = __builtin_amdgcn_exp2f(z);
        part += dead ? 0.0f : term;
        gm = fmaxf(gm, dead ? -INFINITY : x);
        if (WANT_S2) s2[vi][r] = dead ? -INFINITY : z + sc.out_scale;
      } else {
        float v;
        if (CAP) {
          // cap * log2(e) * tanh(x / cap), tanh(u) = 1 - 2 / (1 + exp(2 u))
          const float t = __builtin_amdgcn_exp2f(x * sc.in_scale);
          const float w = __builtin_amdgcn_rcpf(1.0f + t);
          v = fmaf(w, -2.0f * sc.out_scale, sc.out_scale);
        } else {
          v = x;  // the raw logit: the maximum is scaled once per block, the exponent below in its fma
        }
        v = dead ? -INFINITY : v;
        y[vi][r] = v;
        if (WANT_S2) s2[vi][r] = CAP ? v : v * kLog2e;
        gm = fmaxf(gm, v);
      }
    }
    if (!FIXED && !CAP) gm *= kLog2e;
    bm[vi / 2] = fmaxf(bm[vi / 2], gm);
    tm = fmaxf(tm, gm);
  }
  if (FIXED) {
    run.x = sc.out_scale;
    run.y += part;
  } else {
    const float mn = fmaxf(run.x, tm);
    const float ms = (mn == -INFINITY) ? 0.0f : mn;
#pragma unroll
    for (int vi = 0; vi < kF16WV; ++vi)
#pragma unroll
      for (int r = 0; r < 4; ++r) part += __builtin_amdgcn_exp2f(CAP ? y[vi][r] - ms : fmaf(y[vi][r], kLog2e, -ms));
    run.y = run.y * __builtin_amdgcn_exp2f(run.x - ms) + part;
    run.x = mn;
  }
}

// One uniform branch per row block: each arm is straight-line code over all 32 values.
template <bool GENERAL, bool WANT_S2>
__device__ __forceinline__ void row_block(const Softcap& sc, float cap_inv, bool fixed_ref,
                                          const f32x4 (&acc)[kF16WV][kF16WT], int ti,
                                          const float* addend, int kq, float2& run, float (&bm)[kF16WV / 2],
                                          float (&s2)[kF16WV][4]) {
  if (fixed_ref) row_block_impl<GENERAL, true, true, WANT_S2>(sc, cap_inv, acc, ti, addend, kq, run, bm, s2);
  else if (sc.on) row_block_impl<GENERAL, true, false, WANT_S2>(sc, cap_inv, acc, ti, addend, kq, run, bm, s2);
  else row_block_impl<GENERAL, false, false, WANT_S2>(sc, cap_inv, acc, ti, addend, kq, run, bm, s2);
}

template <typename T, bool GENERAL, bool WANT_LA>
__global__ __launch_bounds__(kFwdThreads, 1) void lse_forward16_kernel(LseFwdParams p) {
  using Fast = DmaLogitTile16<T, kF16WV, kF16WT, kFwdNWV, kFwdNWT>;
  static_assert(!WANT_LA || GENERAL, "the column average uses the general epilogue");
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_addend = reinterpret_cast<float*>(smem + Fast::LDS_BYTES);  // [2][256]
  // The running (max, sum-exp) of this lane's kF16WT token rows lives in LDS between the epilogues: [ti][thread].
  // Eight registers fewer across the main loop, which is what lets the loop and the epilogue go without spills
  // (a reload from scratch memory makes the compiler wait for ALL loads in flight, the ring's included).
  float2* s_run = reinterpret_cast<float2*>(smem + Fast::LDS_BYTES + kFwdBiasBytes) + threadIdx.x;
  // WANT_LA: the sums of the soft-capped logits of a tile over its 256 rows, per class: [2][256], by tile parity.
  // The waves add their shares while they are in the epilogue of tile t; the sums leave for memory in the epilogue of
  // tile t + 1 (or after the last tile): the barriers of the main loop in between order the two.
  float* s_colsum = reinterpret_cast<float*>(smem + Fast::LDS_BYTES + kFwdBiasBytes + kF16RunBytes);

  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  if (slot >= p.items_per_xcd) return;
  const int item = xcd * p.items_per_xcd + slot;
  if (item >= p.nitems) return;
  const int rb = item / p.nsplit;
  const int split = item % p.nsplit;
  const int vt_begin = static_cast<int>((static_cast<int64_t>(p.nvt) * split) / p.nsplit);
  const int vt_end = static_cast<int>((static_cast<int64_t>(p.nvt) * (split + 1)) / p.nsplit);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // wave-uniform, and known to the compiler as such: everything derived from it (row and class offsets of the
  // wave, addresses of the statistic cells) then lives in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wv = wave / kFwdNWT;
  const int wt = wave % kFwdNWT;
  const int r16 = lane & 15;
  const int kq = lane >> 4;
  const int64_t t0 = static_cast<int64_t>(rb) * kFwdTile;
  const int64_t wrow0 = t0 + wt * (16 * kF16WT);  // first row of this wave

  // Sources of the direct-to-LDS loads (the launcher has checked that the byte offsets fit 32 bits)
  typename Fast::Source src;
  src.e_base = reinterpret_cast<const unsigned char*>(p.e);
  src.chunk_bytes = 2u * static_cast<unsigned>(Fast::chunk_elems(wave, lane));
  src.row_in_block = static_cast<unsigned>(lane >> 3);
  src.c_stride_bytes = static_cast<unsigned>(p.stride_cv * 2);
#pragma unroll
  for (int q = Fast::NQC; q < Fast::NQ; ++q) {
    int64_t i = t0 + Fast::row_of(q, wave, lane);
    i = (i < p.b) ? i : p.b - 1;  // rows past the end repeat the last one; their results are dropped
    const int64_t row = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
    src.e_off[q - Fast::NQC] = static_cast<unsigned>(row * p.stride_e * 2) + src.chunk_bytes;
  }
  auto set_class_tile = [&](int64_t v0) {
    const int left = static_cast<int>(min(p.v - v0, static_cast<int64_t>(kFwdTile)));  // classes of this tile inside V
    Fast::set_class_tile(src, reinterpret_cast<const unsigned char*>(p.c) + v0 * p.stride_cv * 2, left, wave);
  };

  // 2^(-2 cap log2(e)) must stay a normal float: cap log2(e) < 60, i.e. caps up to 41
  const bool fixed_ref = p.sc.on && p.sc.out_scale < 60.0f;
#pragma unroll
  for (int ti = 0; ti < kF16WT; ++ti) s_run[ti * kFwdThreads] = make_float2(-INFINITY, 0.0f);
  if (WANT_LA) s_colsum[tid] = 0.0f;  // 512 threads, 2 x 256 sums; published by the barriers of the first main loop
  // the sums of the tile that starts at class `first` leave for the running average, and are cleared for the tile after next
  // (the scale comes as a kernel argument and the address is formed where it is used: a lane constant carried
  // through the main loop would be parked in scratch memory, and its reload waits for the loads of the ring)
  auto flush_colsum = [&](int64_t first, int parity) {
    int t = tid;
    asm volatile("" : "+v"(t));
    if (t < kFwdTile) {
      float* cs = s_colsum + parity * kFwdTile + t;
      const float sum = *cs;
      *cs = 0.0f;
      if (first + t < p.v) unsafeAtomicAdd(p.logit_avg + first + t, sum * p.avg_scale);
    }
  };

  float stat = 0.0f;  // statistic cells waiting to be written (see the epilogue)
  int buf = 0;
  set_class_tile(static_cast<int64_t>(vt_begin) * kFwdTile);
  Fast::prefetch(src, smem);

  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int64_t v0 = static_cast<int64_t>(vt) * kFwdTile;
    float* addend = s_addend + (vt & 1) * kFwdTile;
    if (GENERAL) {
      // Written before the main loop, whose barriers publish it; the other buffer may still be read
      // by a wave that is finishing the previous tile.
      if (tid < kFwdTile) {
        const int64_t vg = v0 + tid;
        float a = -INFINITY;
        if (vg < p.v) a = (p.bias != nullptr) ? Elem<T>::to_float(p.bias[vg]) : 0.0f;
        addend[tid] = a;
      }
    }
    f32x4 acc[kF16WV][kF16WT];
    Fast::run(acc, src, smem, static_cast<int>(p.d), buf, vt == vt_begin, [&] {
      if (vt + 1 < vt_end) set_class_tile(v0 + kFwdTile);
    });

    // ---- epilogue: (bias, mask,) soft-cap, online max / sum-exp ---------------------------------
    const float* wave_addend = addend + wv * (16 * kF16WV);
    // A tile with no bias and no class past the end of the vocabulary has nothing to add and nothing to mask: of a
    // vocabulary that is no multiple of 256 only the last tile pays for the per-class addend.
    const bool plain_tile = GENERAL && p.bias == nullptr && v0 + kFwdTile <= p.v;
    float la[WANT_LA ? kF16WV : 1][4];  // this lane's sums over its four rows of the tile, log2 units
    if (WANT_LA) {
      if (vt > vt_begin) flush_colsum(v0 - kFwdTile, (vt - 1) & 1);
#pragma unroll
      for (int vi = 0; vi < kF16WV; ++vi)
#pragma unroll
        for (int r = 0; r < 4; ++r) la[vi][r] = 0.0f;
    }
#pragma unroll
    for (int tp = 0; tp < kF16WT / 2; ++tp) {
      float bm[kF16WV / 2];  // this lane's maxima in the four statistic cells of this row pair
#pragma unroll
      for (int j = 0; j < kF16WV / 2; ++j) bm[j] = -INFINITY;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int ti = 2 * tp + u;
        __builtin_amdgcn_sched_barrier(0);  // keep each row block's register use to itself
        float s2[kF16WV][4];
        float2 run = s_run[ti * kFwdThreads];
        if (GENERAL && plain_tile) row_block<false, WANT_LA>(p.sc, p.cap_inv, fixed_ref, acc, ti, wave_addend, kq, run, bm, s2);
        else row_block<GENERAL, WANT_LA>(p.sc, p.cap_inv, fixed_ref, acc, ti, wave_addend, kq, run, bm, s2);
        s_run[ti * kFwdThreads] = run;
        if (WANT_LA) {
          const bool ok = wrow0 + ti * 16 + r16 < p.b;
#pragma unroll
          for (int vi = 0; vi < kF16WV; ++vi)
#pragma unroll
            for (int r = 0; r < 4; ++r) la[vi][r] += (ok && s2[vi][r] != -INFINITY) ? s2[vi][r] : 0.0f;
        }
      }

      if (p.tile_max != nullptr) {
        // Maxima over the 32 rows x 32 classes of the four statistic cells of this (wave, row pair): wave-uniform
        // values, parked in one register across the lanes -- lane 8 k + 4 tp + j holds cell (row pair tp, class
        // group j) of the k-th tile of a run of eight -- and written out once per eight tiles: a store after every
        // tile would have the next tile's first wait for its loads wait for the store's acknowledgement as well.
        const int slot = (vt - vt_begin) & 7;
#pragma unroll
        for (int j = 0; j < kF16WV / 2; ++j) {
          const float cell = wave_max_uniform(bm[j]);
          stat = (lane == 8 * slot + 4 * tp + j) ? cell : stat;
        }
      }
    }
    if (WANT_LA) {
      // Over the 16 lanes that hold the 16 rows of a block (rotations on the vector unit), then one LDS add per class
      // from the first lane of each group of 16: the four waves that share these classes meet there.
      float* cs = s_colsum + (vt & 1) * kFwdTile + wv * (16 * kF16WV) + 4 * kq;
#pragma unroll
      for (int vi = 0; vi < kF16WV; ++vi)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float sum = row16_sum(la[vi][r]);
          if (r16 == 0) atomicAdd(cs + vi * 16 + r, sum);
        }
    }
    if (p.tile_max != nullptr && (((vt - vt_begin) & 7) == 7 || vt + 1 == vt_end)) {
      int ln = lane;
      if constexpr (WANT_LA) asm volatile("" : "+v"(ln));  // the cell address is formed here, not carried through the loop
      const int first_vt = vt - ((vt - vt_begin) & 7);
      const int my_vt = first_vt + (ln >> 3);
      const int64_t row = wrow0 + ((ln >> 2) & 1) * 32;
      const int64_t cls = static_cast<int64_t>(my_vt) * kFwdTile + wv * (16 * kF16WV) + (ln & 3) * 32;
      if (my_vt <= vt && row < p.b && cls < p.v) {
        float mine = stat;
        if (fixed_ref) {  // the maximum was taken over raw logits
          const float t = __builtin_amdgcn_exp2f(mine * p.sc.in_scale);
          mine = fmaf(__builtin_amdgcn_rcpf(1.0f + t), -2.0f * p.sc.out_scale, p.sc.out_scale);
        }
        p.tile_max[(row / CCE_STAT_ROWS) * p.stat_cols + cls / CCE_STAT_COLS] = mine * kLn2;
      }
    }
  }

  // the loads issued under the last tile (its own first stages once more) must land before the ring is reused
  wait_vmcnt<0>();
  __syncthreads();
  if (WANT_LA && vt_end > vt_begin) flush_colsum(static_cast<int64_t>(vt_end - 1) * kFwdTile, (vt_end - 1) & 1);

  // ---- merge the four lane groups, then the two wave rows, and emit one partial per row -------
  float2* stage = reinterpret_cast<float2*>(smem);  // [NWT][WT][16]
  float m2[kF16WT], sum[kF16WT];
#pragma unroll
  for (int ti = 0; ti < kF16WT; ++ti) {
    const float2 run = s_run[ti * kFwdThreads];
    m2[ti] = run.x;
    sum[ti] = run.y;
  }
#pragma unroll
  for (int ti = 0; ti < kF16WT; ++ti) {
#pragma unroll
    for (int off = 16; off <= 32; off <<= 1) {
      const float om = __shfl_xor(m2[ti], off, 64);
      const float os = __shfl_xor(sum[ti], off, 64);
      const float mn = fmaxf(m2[ti], om);
      const float ms = (mn == -INFINITY) ? 0.0f : mn;
      sum[ti] = sum[ti] * __builtin_amdgcn_exp2f(m2[ti] - ms) + os * __builtin_amdgcn_exp2f(om - ms);
      m2[ti] = mn;
    }
  }
  if (wv == 1 && kq == 0) {
#pragma unroll
    for (int ti = 0; ti < kF16WT; ++ti) stage[(wt * kF16WT + ti) * 16 + r16] = make_float2(m2[ti], sum[ti]);
  }
  __syncthreads();
  if (wv == 0 && kq == 0) {
#pragma unroll
    for (int ti = 0; ti < kF16WT; ++ti) {
      const float2 o = stage[(wt * kF16WT + ti) * 16 + r16];
      const float mn = fmaxf(m2[ti], o.x);
      const float ms = (mn == -INFINITY) ? 0.0f : mn;
      const float s = sum[ti] * __builtin_amdgcn_exp2f(m2[ti] - ms) + o.y * __builtin_amdgcn_exp2f(o.x - ms);
      const int64_t i = wrow0 + ti * 16 + r16;
      if (i < p.b) p.partial[static_cast<int64_t>(split) * p.b + i] = make_float2(mn, s);
    }
  }
}

// lse[i] = ln(2) * (M + log2(sum_s sum_s * 2^(m_s - M))),  M = max_s m_s
__global__ void lse_merge_kernel(const float2* partial, float* lse, int64_t b, int nsplit) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= b) return;
  float m = -INFINITY;
  for (int s = 0; s < nsplit; ++s) m = fmaxf(m, partial[static_cast<int64_t>(s) * b + i].x);
  float acc = 0.0f;
  for (int s = 0; s < nsplit; ++s) {
    const float2 ps = partial[static_cast<int64_t>(s) * b + i];
    acc += ps.y * exp2f(ps.x - m);
  }
  lse[i] = (m + log2f(acc)) * kLn2;
}

__global__ void fill_zero_kernel(float* p, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.0f;
}

static int choose_nsplit(int nrb, int nvt) { return choose_span_count(nrb, nvt); }

template <typename T>
static int launch_lse_forward(LseFwdParams& p, bool aligned, bool want_la, hipStream_t stream) {
  using Tile = LogitTile<T, kFwdWV, kFwdWT, kFwdNWV, kFwdNWT, true>;
  using Fast = DmaLogitTile<T, kFwdWV, kFwdWT, kFwdNWV, kFwdNWT>;
  static_assert(Fast::LDS_BYTES <= Tile::LDS_BYTES, "one LDS size serves both main loops");
  const int lds = Tile::LDS_BYTES + kFwdBiasBytes;
  const int lds16 = lds + kF16RunBytes;  // + the running (max, sum) pairs
  // the 16 x 16 x 32 kernel addresses token rows by 32-bit byte offsets from e and class rows by offsets from the
  // first class of a tile; shapes beyond that, and a D of one stage, take the 32 x 32 x 16 kernel
  const bool fast = aligned && (p.d % kDmaBK == 0);
  const bool fast16 = fast && (p.d >= 2 * kDmaBK) && (p.n_rows * p.stride_e * 2 < (int64_t(1) << 32)) &&
                      (256 * p.stride_cv * 2 < (int64_t(1) << 32));
  const bool general = want_la || (p.bias != nullptr) || (p.v % Tile::TILE_V != 0);
  const int grid = p.items_per_xcd * 8;
  hipError_t err;
#define CCE_LAUNCH_FWD(FA, AL, GE, LA)                                                            \
  do {                                                                                            \
    auto kern = lse_forward_kernel<T, FA, AL, GE, LA>;                                            \
    static LdsLimitOnce lds_limit;                                                            \
    err = lds_limit.set(kern, lds);                                        \
    if (err != hipSuccess) return status_from_hip(err);                                           \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kFwdThreads), lds, stream, p);                           \
  } while (0)
#define CCE_LAUNCH_FWD16(GE, LA)                                                                  \
  do {                                                                                            \
    auto kern = lse_forward16_kernel<T, GE, LA>;                                                  \
    static LdsLimitOnce lds_limit;                                                            \
    const int bytes = lds16 + ((LA) ? kF16ColsumBytes : 0);                                       \
    err = lds_limit.set(kern, bytes);                                                             \
    if (err != hipSuccess) return status_from_hip(err);                                           \
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kFwdThreads), bytes, stream, p);                    \
  } while (0)
  if (fast16) {
    if (want_la) CCE_LAUNCH_FWD16(true, true);
    else if (general) CCE_LAUNCH_FWD16(true, false);
    else CCE_LAUNCH_FWD16(false, false);
  } else if (fast) {
    if (want_la) CCE_LAUNCH_FWD(true, true, true, true);
    else if (general) CCE_LAUNCH_FWD(true, true, true, false);
    else CCE_LAUNCH_FWD(true, true, false, false);
  } else if (aligned) {
    if (want_la) CCE_LAUNCH_FWD(false, true, true, true); else CCE_LAUNCH_FWD(false, true, true, false);
  } else {
    if (want_la) CCE_LAUNCH_FWD(false, false, true, true); else CCE_LAUNCH_FWD(false, false, true, false);
  }
#undef CCE_LAUNCH_FWD
#undef CCE_LAUNCH_FWD16
  return status_from_hip(hipGetLastError());
}

}  // namespace cce

using namespace cce;

extern "C" int64_t cce_tile_stat_elems(int64_t b, int64_t v) {
  if (b <= 0 || v <= 0) return 0;
  return ((b + CCE_STAT_ROWS - 1) / CCE_STAT_ROWS) * ((v + CCE_STAT_COLS - 1) / CCE_STAT_COLS);
}

extern "C" int64_t cce_lse_forward_workspace_bytes(int64_t b, int64_t v, int64_t d) {
  (void)d;
  if (b <= 0 || v <= 0) return 0;
  const int nrb = static_cast<int>((b + 255) / 256);
  const int nvt = static_cast<int>((v + 255) / 256);
  const int nsplit = choose_nsplit(nrb, nvt);
  return static_cast<int64_t>(nsplit) * b * static_cast<int64_t>(sizeof(float2));
}

static int lse_forward_impl(const void* e, const void* c, const void* bias, const int32_t* valids,
                            float* lse, float* logit_avg, float* tile_max,
                            void* workspace, int64_t workspace_bytes,
                            int64_t n_rows, int64_t b, int64_t v, int64_t d,
                            int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                            float softcap, int dtype, hipStream_t stream) {
  const int64_t need = cce_lse_forward_workspace_bytes(b, v, d);
  if (workspace == nullptr || workspace_bytes < need) return CCE_ERR_WORKSPACE_TOO_SMALL;
  if ((reinterpret_cast<uintptr_t>(workspace) & 7u) != 0) return CCE_ERR_MISALIGNED;

  LseFwdParams p;
  p.e = static_cast<const uint16_t*>(e);
  p.c = static_cast<const uint16_t*>(c);
  p.bias = static_cast<const uint16_t*>(bias);
  p.valids = valids;
  p.logit_avg = logit_avg;
  p.tile_max = tile_max;
  p.partial = static_cast<float2*>(workspace);
  p.b = b;
  p.v = v;
  p.d = d;
  p.n_rows = n_rows;
  p.stride_e = stride_e;
  p.stride_cv = stride_cv;
  p.stride_cd = stride_cd;
  p.nrb = static_cast<int>((b + 255) / 256);
  p.nvt = static_cast<int>((v + 255) / 256);
  p.nsplit = choose_nsplit(p.nrb, p.nvt);
  p.nitems = p.nrb * p.nsplit;
  p.items_per_xcd = (p.nitems + 7) / 8;
  p.stat_cols = static_cast<int>((v + CCE_STAT_COLS - 1) / CCE_STAT_COLS);
  p.avg_scale = kLn2 / static_cast<float>(b);
  p.sc = make_softcap(softcap);
  p.cap_inv = p.sc.on ? 1.0f / (-2.0f * p.sc.out_scale) : 0.0f;

  const bool aligned = aligned16(e) && aligned16(c) && (d % 8 == 0) && (stride_e % 8 == 0) &&
                       (stride_cv % 8 == 0) && (stride_cd == 1);

  if (logit_avg != nullptr) {
    hipLaunchKernelGGL(fill_zero_kernel, dim3(static_cast<unsigned>((v + 255) / 256)), dim3(256), 0, stream,
                       logit_avg, v);
  }
  int st = (dtype == CCE_DTYPE_BF16) ? launch_lse_forward<BF16>(p, aligned, logit_avg != nullptr, stream)
                                     : launch_lse_forward<F16>(p, aligned, logit_avg != nullptr, stream);
  if (st != CCE_OK) return st;
  hipLaunchKernelGGL(lse_merge_kernel, dim3(static_cast<unsigned>((b + 255) / 256)), dim3(256), 0, stream,
                     p.partial, lse, b, p.nsplit);
  return status_from_hip(hipGetLastError());
}

// Argument checks shared by the two entry points; CCE_OK with *done set means "nothing to do".
static int lse_forward_check(const void* e, const void* c, const float* lse, const int32_t* valids,
                             int64_t n_rows, int64_t b, int64_t v, int64_t d, int dtype, bool* done) {
  *done = false;
  if (b < 0 || v <= 0 || d <= 0 || n_rows < 0) return CCE_ERR_INVALID_ARGUMENT;
  if (b == 0) {
    *done = true;
    return CCE_OK;
  }
  if (e == nullptr || c == nullptr || lse == nullptr) return CCE_ERR_INVALID_ARGUMENT;
  if (valids == nullptr && b > n_rows) return CCE_ERR_INVALID_ARGUMENT;
  if (d > (1 << 30) || b > (int64_t(1) << 40) || v > (int64_t(1) << 31) - 512) return CCE_ERR_INVALID_ARGUMENT;
  if (dtype != CCE_DTYPE_BF16 && dtype != CCE_DTYPE_F16) return CCE_ERR_UNSUPPORTED_DTYPE;
  return CCE_OK;
}

extern "C" int cce_lse_forward(const void* e, const void* c, const void* bias, const int32_t* valids,
                               float* lse, float* logit_avg, float* tile_max,
                               void* workspace, int64_t workspace_bytes,
                               int64_t n_rows, int64_t b, int64_t v, int64_t d,
                               int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                               float softcap, int dtype, void* stream_) {
  bool done;
  const int st = lse_forward_check(e, c, lse, valids, n_rows, b, v, d, dtype, &done);
  if (st != CCE_OK || done) return st;
  return lse_forward_impl(e, c, bias, valids, lse, logit_avg, tile_max, workspace, workspace_bytes, n_rows, b, v, d,
                          stride_e, stride_cv, stride_cd, softcap, dtype, static_cast<hipStream_t>(stream_));
}

// ---------------------------------------------------------------------------------------------
// The same forward for callers that may not allocate: the split-vocabulary partials live in a
// file-scope device array instead of a caller's workspace.  Each GPU holds its own copy of the
// array, at its own address, until the process ends; the address is looked up once per device (with
// that device current) and from then on only that pointer is used -- the array's name is a host-side
// handle, not a device address.  Every (span, row) partial a launch reads is written by the same
// launch first, so nothing has to be cleared between calls; calls that overlap on one GPU (two
// streams, two threads) share the array and race.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[CCE_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
}  // namespace

static int static_scratch_for_current_device(void** out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return status_from_hip(err);
  if (dev < 0 || dev >= kMaxDevices) return CCE_ERR_INVALID_ARGUMENT;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return status_from_hip(err);
    if (ptr == nullptr) return CCE_ERR_INVALID_ARGUMENT;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // every thread finds the same address
  }
  *out = ptr;
  return CCE_OK;
}

extern "C" int cce_lse_forward_static_init(void) {
  void* ws = nullptr;
  return static_scratch_for_current_device(&ws);
}

extern "C" int cce_lse_forward_static(const void* e, const void* c, const void* bias, const int32_t* valids,
                                      float* lse, float* logit_avg, float* tile_max,
                                      int64_t n_rows, int64_t b, int64_t v, int64_t d,
                                      int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                                      float softcap, int dtype, void* stream_) {
  bool done;
  int st = lse_forward_check(e, c, lse, valids, n_rows, b, v, d, dtype, &done);
  if (st != CCE_OK || done) return st;
  if (cce_lse_forward_workspace_bytes(b, v, d) > CCE_STATIC_SCRATCH_BYTES) return CCE_ERR_STATIC_SCRATCH_LIMIT;
  void* ws = nullptr;
  st = static_scratch_for_current_device(&ws);
  if (st != CCE_OK) return st;
  return lse_forward_impl(e, c, bias, valids, lse, logit_avg, tile_max, ws, CCE_STATIC_SCRATCH_BYTES, n_rows, b, v, d,
                          stride_e, stride_cv, stride_cd, softcap, dtype, static_cast<hipStream_t>(stream_));
}
