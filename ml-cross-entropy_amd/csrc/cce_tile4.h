// One 256 x 256 tile of  Out[m][n] = sum_k A[m][k] * B[k][n]  on one compute unit with FOUR waves, one per
// SIMD, each owning 128 x 128 of the tile: 4 x 4 accumulator blocks of 32 x 32 = 256 accumulation registers.
// Per 16 reduction steps a wave reads 4 + 4 operand fragments for 16 MFMAs -- two thirds of the LDS reads per
// MFMA of a 2 x 4 arrangement of eight waves (6 for 8).  With one wave per SIMD nothing else hides a wave's own
// instruction issue: an MFMA occupies the matrix pipeline for 32 cycles, and whatever the wave issues between two
// of them beyond ~28 cycles idles the pipeline.  The main loop is therefore kept lean: every LDS address is a
// per-lane base plus an immediate, the address of a load is a per-lane base plus an offset the scalar unit forms
// (one vector instruction), and nothing inside the loop asks whether a row exists.
//
// Either operand is streamed through LDS by direct global -> LDS loads (`global_load_lds_dwordx4`), in one
// of two layouts:
//   Direct   the operand's rows are tile rows (m or n) and the reduction index is contiguous in memory:
//            LDS image 256 rows x 128 bytes (64 k), 16-byte chunks XOR-swizzled with (row >> 1) & 7; one load
//            instruction fills 8 rows; a fragment is one 16-byte read.
//   KMajor   the matrix is [K][256] row-major (reduction index = row): LDS image 64 rows x 512 bytes, the 32
//            chunks of a row XOR-swizzled with 4 (row & 3); one load instruction fills 2 rows (lanes 0-31 one,
//            lanes 32-63 the next); a fragment is two LDS transpose reads (`ds_read_b64_tr_b16`) of four k rows
//            each.  In one such read a group of 16 lanes supplies 16 addresses of 4 elements -- lane i: row
//            r0 + (i >> 2), columns c0 + 4 (i & 3) .. + 3 -- and lane i receives the elements [r0 .. r0 + 3][c0 + i].
//            The rows of a KMajor B may be gathered through an index vector (B_GATHER): a lane looks its row
//            number up with one load (uniform base + (lane >> 5)) a step ahead and forms the address with one
//            multiply-add.
// A column chunk past the matrix is fetched from the last chunk inside it instead (it only feeds outputs the
// caller drops).  A reduction that is not a multiple of 64 has one partial stage: it is the FIRST stage of the
// tile, fetched before the main loop by loads that ask per row whether the row exists and take a line of zeros
// when not, so that a non-finite value elsewhere never meets the product; the loop then walks whole stages
// only, and what it fetches past the end of the reduction (its loads run two stages ahead) is the last whole
// stage again, never consumed.
//
// A stage is 64 reduction steps (32 KB per operand), two stages per operand in LDS (operand-major: A0 A1 B0 B1,
// so that every read offset fits the 16-bit immediate), one barrier per stage.  The loads of a stage are
// issued in two groups of 8, one load after every second MFMA: A under the last 16-step of the stage before last,
// B under the first 16-step of the stage before; the fragment reads of step k + 1 go out between the MFMAs of
// step k.  Completion of the loads is tracked by hand (s_waitcnt vmcnt), the compiler cannot see them.
#pragma once

#include <utility>

#include "cce_common.h"

namespace cce {

static __device__ __align__(256) uint16_t g_zero_line[128];  // never written

typedef short tr_short4_t __attribute__((ext_vector_type(4)));

template <typename T, bool A_KM, bool B_KM, bool B_GATHER = false>
struct Tile4 {
  static_assert(!B_GATHER || B_KM, "only the rows of a KMajor operand are gathered");
  static constexpr int WM = 4, WN = 4;   // accumulator blocks per wave
  static constexpr int NW = 4;           // waves, 2 (m) x 2 (n)
  static constexpr int NT = 64 * NW;
  static constexpr int TILE = 256;
  static constexpr int BK = 64;
  static constexpr int OP_BYTES = 32 * 1024;      // one stage of one operand
  static constexpr int B_BASE = 2 * OP_BYTES;     // A stage 0, A stage 1, B stage 0, B stage 1
  static constexpr int LDS_BYTES = 4 * OP_BYTES;
  static constexpr int NQ1 = 8;          // loads per wave, stage and operand
  using vec8 = typename Elem<T>::vec8;

  // ---- what a lane fetches ---------------------------------------------------------------------------
  static __device__ __forceinline__ int row_direct(int q, int wave, int lane) { return 8 * (q * NW + wave) + (lane >> 3); }
  static __device__ __forceinline__ int chunk_direct(int wave, int lane) {
    const int sw = (4 * (wave & 1) + (lane >> 4)) & 7;  // (row >> 1) & 7
    return ((lane & 7) ^ sw) * 8;
  }
  // KMajor: load q of a wave covers stage rows 2 (q NW + wave) and the next; this lane's is the (lane >> 5)-th
  static __device__ __forceinline__ int row_kmajor(int q, int wave) { return 2 * (q * NW + wave); }
  static __device__ __forceinline__ int chunk_kmajor(int wave, int lane) {
    const int r3 = (2 * (wave & 1) + (lane >> 5)) & 3;  // row & 3
    return ((lane & 31) ^ (r3 << 2)) * 8;
  }

  struct Source {
    const uint16_t* a_row[A_KM ? 1 : NQ1];  // Direct: row base + chunk_direct, one row per load
    const uint16_t* b_row[B_KM ? 1 : NQ1];
    const uint16_t* a_km;   // KMajor: matrix base + first column of the tile + chunk_kmajor, inside the matrix
    const uint16_t* b_km;
    int64_t a_stride;       // KMajor: elements between consecutive k rows (< 2^30)
    int64_t b_stride;
    const int32_t* b_rows;  // B_GATHER: the k rows of B (k_total entries)
    int k_total;            // length of the reduction
  };

  // What the loads inside the main loop work from (built by plan()).  With no whole stage in the reduction the
  // loop still issues its loads: they then read the line of zeros (stride 0, row numbers from the same line).
  struct Loop {
    const uint16_t* a_lane;  // KMajor: this lane's address in rows 0 / 1 of the matrix (a_km + (lane >> 5) stride)
    const uint16_t* b_lane;  //   (a gathered B: without the row term)
    uint32_t a_stride, b_stride;
    const int32_t* b_rows;
    int nk;          // stages
    int partial;     // 1: stage 0 is the partial last 64-step of the reduction, stage t >= 1 is whole stage t - 1
    int k_first;     // where stage 0 starts
    int k_clamp;     // where the last whole stage starts
  };

  // Per-lane constants of the main loop.
  struct Geometry {
    int lane, wave, wm, wn, l32, half;
    unsigned lds_base;
    // LDS byte addresses (inside a stage) of this lane's fragment reads
    int a_addr[4];  // Direct: one per 16-step kk (block i adds i * 4096); KMajor: one per block i (kk adds kk * 8192)
    int b_addr[4];
  };
  static __device__ __forceinline__ Geometry geometry(unsigned char* lds) {
    Geometry g;
    g.lane = threadIdx.x & 63;
    g.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    g.wm = g.wave >> 1;
    g.wn = g.wave & 1;
    g.l32 = g.lane & 31;
    g.half = g.lane >> 5;
    g.lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));
    const int sw = (g.l32 >> 1) & 7;
    const int tr_row = 8 * (g.lane >> 5) + ((g.lane >> 2) & 3);
    const int tr_col = 16 * ((g.lane >> 4) & 1) + 4 * (g.lane & 3);
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      if (A_KM) {
        const int col = g.wm * 128 + x * 32 + tr_col;
        g.a_addr[x] = tr_row * 512 + ((((col >> 3) ^ ((tr_row & 3) << 2)) << 4) | ((col & 7) << 1));
      } else {
        g.a_addr[x] = (g.wm * 128 + g.l32) * 128 + (((x * 2 + g.half) ^ sw) << 4);
      }
      if (B_KM) {
        const int col = g.wn * 128 + x * 32 + tr_col;
        g.b_addr[x] = B_BASE + tr_row * 512 + ((((col >> 3) ^ ((tr_row & 3) << 2)) << 4) | ((col & 7) << 1));
      } else {
        g.b_addr[x] = B_BASE + (g.wn * 128 + g.l32) * 128 + (((x * 2 + g.half) ^ sw) << 4);
      }
    }
    return g;
  }

  static __device__ __forceinline__ const uint16_t* zero_line(const Geometry& g) { return g_zero_line + (g.lane & 15) * 8; }

  static __device__ __forceinline__ Loop plan(const Source& s, const Geometry& g) {
    Loop l;
    const int whole = s.k_total / BK;
    l.partial = (s.k_total % BK) != 0;
    l.nk = whole + l.partial;
    l.k_first = l.partial ? whole * BK : 0;
    l.k_clamp = whole > 0 ? (whole - 1) * BK : 0;
    const bool any = whole > 0;
    l.a_stride = any ? static_cast<uint32_t>(s.a_stride) : 0u;
    l.b_stride = any ? static_cast<uint32_t>(s.b_stride) : 0u;
    l.a_lane = zero_line(g);
    l.b_lane = zero_line(g);
    if (A_KM && any) l.a_lane = s.a_km + static_cast<uint32_t>(g.half) * l.a_stride;
    if (B_KM && any) l.b_lane = B_GATHER ? s.b_km : s.b_km + static_cast<uint32_t>(g.half) * l.b_stride;
    l.b_rows = (B_GATHER && any) ? s.b_rows : reinterpret_cast<const int32_t*>(g_zero_line);
    return l;
  }
  // Where stage t >= 1 starts; past the end of the reduction: the last whole stage again.
  static __device__ __forceinline__ int k_of(const Loop& l, int t) { return min((t - l.partial) * BK, l.k_clamp); }

  // The row numbers and load addresses of a gathered B, formed a step ahead of their use.
  struct Ids {
    int v[B_GATHER ? NQ1 : 1];
  };
  struct Ptrs {
    const uint16_t* b[B_GATHER ? NQ1 : 1];
  };

  // ---- loads inside the main loop: whole stages only, nothing is checked ------------------------------
  static __device__ __forceinline__ void prep_b_id(Ids& ids, int q, const Loop& l, int k0, const Geometry& g) {
    if (!B_GATHER) return;
    const int32_t* pair = l.b_rows + (k0 + row_kmajor(q, g.wave));  // uniform
    ids.v[B_GATHER ? q : 0] = pair[g.half];
  }
  static __device__ __forceinline__ void prep_b(Ptrs& p, int q, const Ids& ids, const Loop& l, const Geometry&) {
    if (!B_GATHER) return;
    p.b[B_GATHER ? q : 0] = l.b_lane + static_cast<uint64_t>(static_cast<uint32_t>(ids.v[B_GATHER ? q : 0])) * l.b_stride;
  }
  // Load q of the stage that starts at k0 (a whole stage) into LDS stage STAGE.
  template <int STAGE>
  static __device__ __forceinline__ void issue_a(int q, const Source& s, const Loop& l, int k0, const Geometry& g) {
    const uint16_t* src;
    if (A_KM) {
      const uint32_t r = static_cast<uint32_t>(k0 + row_kmajor(q, g.wave));  // uniform
      src = l.a_lane + static_cast<uint64_t>(r) * l.a_stride;
    } else {
      src = s.a_row[A_KM ? 0 : q] + k0;
    }
    lds_dma16(src, g.lds_base + STAGE * OP_BYTES + (q * NW + g.wave) * 1024);
  }
  template <int STAGE>
  static __device__ __forceinline__ void issue_b(const Ptrs& p, int q, const Source& s, const Loop& l, int k0,
                                                const Geometry& g) {
    const uint16_t* src;
    if (B_GATHER) {
      src = p.b[B_GATHER ? q : 0];
    } else if (B_KM) {
      const uint32_t r = static_cast<uint32_t>(k0 + row_kmajor(q, g.wave));  // uniform
      src = l.b_lane + static_cast<uint64_t>(r) * l.b_stride;
    } else {
      src = s.b_row[B_KM ? 0 : q] + k0;
    }
    lds_dma16(src, g.lds_base + B_BASE + STAGE * OP_BYTES + (q * NW + g.wave) * 1024);
  }

  // ---- loads of stage 0 (the partial stage when there is one): every row is asked for --------------------
  static __device__ __forceinline__ void issue_first_a(int q, const Source& s, int k0, const Geometry& g) {
    const uint16_t* src;
    if (A_KM) {
      const int row = k0 + row_kmajor(q, g.wave) + g.half;
      src = s.a_km + static_cast<uint64_t>(static_cast<uint32_t>(row)) * static_cast<uint32_t>(s.a_stride);
      if (row >= s.k_total) src = zero_line(g);
    } else {
      src = s.a_row[A_KM ? 0 : q] + k0;
    }
    lds_dma16(src, g.lds_base + (q * NW + g.wave) * 1024);
  }
  // (the row numbers of a gathered B are looked up for all loads first: the lookups and the loads share a queue)
  static __device__ __forceinline__ int first_b_id(int q, const Source& s, int k0, const Geometry& g) {
    if (!B_KM) return 0;
    const int row = k0 + row_kmajor(q, g.wave) + g.half;
    int id = -1;
    if (row < s.k_total) id = B_GATHER ? s.b_rows[row] : row;
    return id;
  }
  static __device__ __forceinline__ void issue_first_b(int q, int id, const Source& s, int k0, const Geometry& g) {
    const uint16_t* src;
    if (B_KM) {
      src = s.b_km + static_cast<uint64_t>(static_cast<uint32_t>(id)) * static_cast<uint32_t>(s.b_stride);
      if (id < 0) src = zero_line(g);
    } else {
      src = s.b_row[B_KM ? 0 : q] + k0;
    }
    lds_dma16(src, g.lds_base + B_BASE + (q * NW + g.wave) * 1024);
  }

  // ---- fragment reads --------------------------------------------------------------------------------
  struct Frags {
    vec8 a[WM];
    vec8 b[WN];
  };
  struct Half {
    tr_short4_t lo, hi;
  };
  static __device__ __forceinline__ tr_short4_t read_tr(const unsigned char* lds, int addr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) tr_short4_t*)(lds + addr));
  }
  static __device__ __forceinline__ vec8 read_16(const unsigned char* lds, int addr) {
    return __builtin_bit_cast(vec8, *reinterpret_cast<const uint4*>(lds + addr));
  }
  static constexpr int kReadsA = A_KM ? 2 : 1;
  static constexpr int kReadsB = B_KM ? 2 : 1;
  static constexpr int kReads = WM * kReadsA + WN * kReadsB;
  // part `part` of the read of fragment a[i] / b[i] of step KK of stage STAGE: the address is a lane constant
  // plus a compile-time offset below 64 K.
  template <int STAGE, int KK>
  static __device__ __forceinline__ void read_a(int i, int part, Frags& f, Half (&h)[WM], const unsigned char* lds,
                                                const Geometry& g) {
    if (A_KM) {
      const tr_short4_t v = read_tr(lds, g.a_addr[i] + STAGE * OP_BYTES + KK * 16 * 512 + part * 4 * 512);
      if (part) h[i].hi = v; else h[i].lo = v;
      if (part) f.a[i] = __builtin_bit_cast(vec8, h[i]);
    } else {
      f.a[i] = read_16(lds, g.a_addr[KK] + STAGE * OP_BYTES + i * 32 * 128);
    }
  }
  template <int STAGE, int KK>
  static __device__ __forceinline__ void read_b(int i, int part, Frags& f, Half (&h)[WN], const unsigned char* lds,
                                                const Geometry& g) {
    if (B_KM) {
      const tr_short4_t v = read_tr(lds, g.b_addr[i] + STAGE * OP_BYTES + KK * 16 * 512 + part * 4 * 512);
      if (part) h[i].hi = v; else h[i].lo = v;
      if (part) f.b[i] = __builtin_bit_cast(vec8, h[i]);
    } else {
      f.b[i] = read_16(lds, g.b_addr[KK] + STAGE * OP_BYTES + i * 32 * 128);
    }
  }
  // Read op r of a step, in the order the MFMAs (m-major) want their operands: a0, b0 .. b3, a1, a2, a3.
  template <int STAGE, int KK>
  static __device__ __forceinline__ void read_op(int r, Frags& f, Half (&ha)[WM], Half (&hb)[WN], const unsigned char* lds,
                                                 const Geometry& g) {
    if (r < kReadsA) {
      read_a<STAGE, KK>(0, r, f, ha, lds, g);
    } else if (r < kReadsA + WN * kReadsB) {
      const int j = r - kReadsA;
      read_b<STAGE, KK>(j / kReadsB, j % kReadsB, f, hb, lds, g);
    } else {
      const int j = r - kReadsA - WN * kReadsB;
      read_a<STAGE, KK>(1 + j / kReadsA, j % kReadsA, f, ha, lds, g);
    }
  }
  template <int STAGE, int KK>
  static __device__ __forceinline__ void read_all(Frags& f, const unsigned char* lds, const Geometry& g) {
    Half ha[WM], hb[WN];
#pragma unroll
    for (int r = 0; r < kReads; ++r) read_op<STAGE, KK>(r, f, ha, hb, lds, g);
  }

  // What a 16-step does between its MFMAs besides the fragment reads of the next step:
  //   kIssueB  + loads of B for the stage at kl into LDS stage LSTAGE, one after every odd MFMA
  //   kPrepIds + row numbers of a gathered B for the stage at k0, one pair after every even MFMA
  //   kIssueAPrepB  loads of A for the stage at kl into LDS stage LSTAGE after the odd MFMAs, addresses of the
  //                 loads of a gathered B (from `ids`) after the even ones
  enum Extra { kNone, kIssueB, kPrepIds, kIssueAPrepB };

  // The 16 MFMAs on `cur`; between them the reads of fragment set `nxt` (step RKK of stage RSTAGE) and EXTRA.
  template <int RSTAGE, int RKK, Extra EXTRA, int LSTAGE>
  static __device__ __forceinline__ void step(f32x16 (&acc)[WM][WN], const Frags& cur, Frags& nxt, const unsigned char* lds,
                                              const Source& s, const Loop& l, int kl, int k0, Ptrs& ptrs, Ids& ids,
                                              const Geometry& g) {
    constexpr int kMfmas = WM * WN;
    Half ha[WM], hb[WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        acc[i][j] = Elem<T>::mfma(cur.a[i], cur.b[j], acc[i][j]);
        const int idx = i * WN + j;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = idx * kReads / kMfmas; r < (idx + 1) * kReads / kMfmas; ++r)
          read_op<RSTAGE, RKK>(r, nxt, ha, hb, lds, g);
        const int q = idx >> 1;
        if (idx & 1) {
          if (EXTRA == kIssueB) issue_b<LSTAGE>(ptrs, q, s, l, kl, g);
          if (EXTRA == kIssueAPrepB) issue_a<LSTAGE>(q, s, l, kl, g);
        } else {
          if (EXTRA == kPrepIds) prep_b_id(ids, q, l, k0, g);
          if (EXTRA == kIssueAPrepB) prep_b(ptrs, q, ids, l, g);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
  }

  // Start fetching a tile into the idle LDS ring: all of stage 0 and the A loads of stage 1; leaves in `ptrs`
  // the addresses of a gathered B for stage 1.  A caller with work between two tiles (an epilogue) calls this
  // first, so that the next main loop starts with data in LDS.
  static __device__ __forceinline__ void prefetch(const Source& s, const Loop& l, Ptrs& ptrs, Ids& ids, const Geometry& g) {
    int first[NQ1];
#pragma unroll
    for (int q = 0; q < NQ1; ++q) first[q] = first_b_id(q, s, l.k_first, g);
#pragma unroll
    for (int q = 0; q < NQ1; ++q) issue_first_a(q, s, l.k_first, g);
#pragma unroll
    for (int q = 0; q < NQ1; ++q) issue_first_b(q, first[q], s, l.k_first, g);
    const int k1 = k_of(l, 1);
#pragma unroll
    for (int q = 0; q < NQ1; ++q) prep_b_id(ids, q, l, k1, g);
#pragma unroll
    for (int q = 0; q < NQ1; ++q) issue_a<1>(q, s, l, k1, g);
#pragma unroll
    for (int q = 0; q < NQ1; ++q) prep_b(ptrs, q, ids, l, g);
  }

  // One stage (four 16-steps) whose data sits in LDS stage CUR; `fa` holds its first fragment set on entry and
  // that of the next stage on exit.
  template <int CUR>
  static __device__ __forceinline__ void stage(f32x16 (&acc)[WM][WN], Frags& fa, Frags& fb, const unsigned char* lds,
                                               const Source& s, const Loop& l, int st, Ptrs& ptrs, Ids& ids,
                                               const Geometry& g) {
    constexpr int NXT = 1 - CUR;
    const int k1 = k_of(l, st + 1);
    const int k2 = k_of(l, st + 2);
    step<CUR, 1, kIssueB, NXT>(acc, fa, fb, lds, s, l, k1, k2, ptrs, ids, g);    // the B loads of stage st + 1
    step<CUR, 2, kPrepIds, NXT>(acc, fb, fa, lds, s, l, k1, k2, ptrs, ids, g);   // rows of B for stage st + 2
    step<CUR, 3, kNone, NXT>(acc, fa, fb, lds, s, l, k1, k2, ptrs, ids, g);
    // Stage st + 1 has landed for this wave; after the barrier for every wave, and every wave holds its last
    // fragments of stage st in registers: that LDS stage is free for stage st + 2.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (B_GATHER) {
      // The looked-up rows are pinned as used here, where nothing is in flight: the compiler places its own
      // wait for them at their first use, and further down it would also wait for the direct-to-LDS loads.
#pragma unroll
      for (int q = 0; q < NQ1; ++q) asm volatile("" : "+v"(ids.v[q]));
    }
    __syncthreads();
    step<NXT, 0, kIssueAPrepB, CUR>(acc, fb, fa, lds, s, l, k2, k2, ptrs, ids, g);  // the A loads of stage st + 2
  }

  // Every per-lane value the main loop reads, marked as used: should the compiler have parked one of them in
  // scratch memory around the caller's code, it reloads it (and waits for that load) here, and not inside the
  // loop, where its wait would also wait for the direct-to-LDS loads in flight, stage after stage.
  static __device__ __forceinline__ void pin(Source& s, Loop& l, Ptrs& ptrs, Geometry& g) {
#pragma unroll
    for (int q = 0; q < (A_KM ? 1 : NQ1); ++q) asm volatile("" : "+v"(s.a_row[q]));
#pragma unroll
    for (int q = 0; q < (B_KM ? 1 : NQ1); ++q) asm volatile("" : "+v"(s.b_row[q]));
#pragma unroll
    for (int q = 0; q < (B_GATHER ? NQ1 : 1); ++q) asm volatile("" : "+v"(ptrs.b[q]));
    if (A_KM) asm volatile("" : "+v"(l.a_lane));
    if (B_KM) asm volatile("" : "+v"(l.b_lane));
#pragma unroll
    for (int x = 0; x < 4; ++x) asm volatile("" : "+v"(g.a_addr[x]), "+v"(g.b_addr[x]));
  }

  // acc = A . B over the whole reduction.  prefetch() with the same source must have been called and nothing
  // may have touched the LDS ring since.  Ends with a barrier: the LDS may be reused right after.
  static __device__ __forceinline__ void run(f32x16 (&acc)[WM][WN], Source& s, Loop& l, Ptrs& ptrs, Ids& ids,
                                             unsigned char* lds, Geometry& g) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int nk = l.nk;
    // stage 0 has landed, the A loads of stage 1 may be in flight (the row lookups of stage 0 of a gathered B sit
    // ahead of its loads in the same queue and are covered by the same count)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NQ1) : "memory");
    pin(s, l, ptrs, g);
    __syncthreads();
    Frags fa, fb;
    read_all<0, 0>(fa, lds, g);

    // two stages per trip, so that every LDS address is a lane constant plus an immediate; an odd last stage
    // stands outside the loop (a branch inside it costs the register allocator its footing)
#pragma unroll 1
    for (int st = 0; st + 1 < nk; st += 2) {
      stage<0>(acc, fa, fb, lds, s, l, st, ptrs, ids, g);
      stage<1>(acc, fa, fb, lds, s, l, st + 1, ptrs, ids, g);
    }
    if (nk & 1) stage<0>(acc, fa, fb, lds, s, l, nk - 1, ptrs, ids, g);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the last, unused prefetch
    __syncthreads();
  }

  // ---- the finished tile, as row pieces ----------------------------------------------------------------
  // The accumulators hold the tile with its columns along the lanes: written out as they are, a lane would
  // touch one element (2 or 4 bytes) of 16 rows.  Each wave instead passes its 128 x 128 part through LDS (idle
  // after run()), 32 rows x 64 columns at a time, and hands `f` pieces of 8 consecutive columns of one row:
  //     f(row, col, v)   row, col: position inside the 256 x 256 tile; v[8]: the values [row][col .. col + 7]
  // so that a piece is one 16-byte (16-bit data) or two 16-byte (fp32) accesses and 8 lanes cover 128 or 256
  // contiguous bytes of a row.  The staging area is private to the wave: no barrier.
  static constexpr int kPieceCols = 8;
  static constexpr int kStagePitch = (64 + 4) * 4;           // bytes per staged row
  static constexpr int kStageBytes = 32 * kStagePitch;       // per wave
  static_assert(NW * kStageBytes <= LDS_BYTES, "the staging areas reuse the ring");

  template <typename F>
  static __device__ __forceinline__ void for_each_row_piece(f32x16 (&acc)[WM][WN], unsigned char* lds, const Geometry& g,
                                                            F&& f) {
    unsigned char* stage = lds + g.wave * kStageBytes;
    static_for<WM * (WN / 2)>([&](auto ij) {
      constexpr int i = decltype(ij)::value / (WN / 2);
      constexpr int jp = decltype(ij)::value % (WN / 2);
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = 8 * (r >> 2) + 4 * g.half + (r & 3);
          *reinterpret_cast<float*>(stage + m * kStagePitch + (jj * 32 + g.l32) * 4) = acc[i][jp * 2 + jj][r];
        }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int pass = 0; pass < 4; ++pass) {
        const int m = pass * 8 + (g.lane >> 3);
        const int c8 = (g.lane & 7) * kPieceCols;
        const float4 lo = *reinterpret_cast<const float4*>(stage + m * kStagePitch + c8 * 4);
        const float4 hi = *reinterpret_cast<const float4*>(stage + m * kStagePitch + c8 * 4 + 16);
        const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        f(g.wm * 128 + i * 32 + m, g.wn * 128 + jp * 64 + c8, v);
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the reads are done before the next slab is staged
    });
  }

  // The same for an output that is combined with what memory holds (dE is summed over the chunks): `fetch(row,
  // col)` returns what `store(row, col, v, old)` needs of the old contents.  The fetches of a slab are issued two
  // slabs ahead (a slab takes about a microsecond, a load under this traffic up to two, two dependent ones where
  // the rows are gathered), those of the first two slabs by rmw_begin() right before, so that their latency is paid
  // once per tile and not once per slab.
  static constexpr int kSlabs = WM * (WN / 2);
  static constexpr int kAhead = 2;
  template <typename Old>
  struct Rmw {
    Old old[kAhead + 1][4];
  };
  template <int SLAB, typename Old, typename Fetch>
  static __device__ __forceinline__ void rmw_fetch(Rmw<Old>& r, const Geometry& g, Fetch&& fetch) {
    constexpr int i = SLAB / (WN / 2);
    constexpr int jp = SLAB % (WN / 2);
#pragma unroll
    for (int pass = 0; pass < 4; ++pass)
      r.old[SLAB % (kAhead + 1)][pass] =
          fetch(g.wm * 128 + i * 32 + pass * 8 + (g.lane >> 3), g.wn * 128 + jp * 64 + (g.lane & 7) * kPieceCols);
  }
  template <typename Old, typename Fetch>
  static __device__ __forceinline__ void rmw_begin(Rmw<Old>& r, const Geometry& g, Fetch&& fetch) {
    static_for<kAhead>([&](auto slab) { rmw_fetch<decltype(slab)::value>(r, g, fetch); });
  }
  template <typename Old, typename Fetch, typename Store>
  static __device__ __forceinline__ void for_each_row_piece_rmw(f32x16 (&acc)[WM][WN], unsigned char* lds, const Geometry& g,
                                                                Rmw<Old>& r, Fetch&& fetch, Store&& store) {
    unsigned char* stage = lds + g.wave * kStageBytes;
    const int c8 = (g.lane & 7) * kPieceCols;
    const int m_lane = g.lane >> 3;
    static_for<kSlabs>([&](auto ij) {
      constexpr int i = decltype(ij)::value / (WN / 2);
      constexpr int jp = decltype(ij)::value % (WN / 2);
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int rr = 0; rr < 16; ++rr) {
          const int m = 8 * (rr >> 2) + 4 * g.half + (rr & 3);
          *reinterpret_cast<float*>(stage + m * kStagePitch + (jj * 32 + g.l32) * 4) = acc[i][jp * 2 + jj][rr];
        }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if constexpr (decltype(ij)::value + kAhead < kSlabs) rmw_fetch<decltype(ij)::value + kAhead>(r, g, fetch);
#pragma unroll
      for (int pass = 0; pass < 4; ++pass) {
        const int m = pass * 8 + m_lane;
        const float4 lo = *reinterpret_cast<const float4*>(stage + m * kStagePitch + c8 * 4);
        const float4 hi = *reinterpret_cast<const float4*>(stage + m * kStagePitch + c8 * 4 + 16);
        const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        store(g.wm * 128 + i * 32 + m, g.wn * 128 + jp * 64 + c8, v, r.old[decltype(ij)::value % (kAhead + 1)][pass]);
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the reads are done before the next slab is staged
    });
  }
};

}  // namespace cce
