// Shared device code of the gfx950 Cut Cross-Entropy kernels: element types, MFMA wrappers,
// the global -> LDS tile loader and the LDS -> MFMA logit-tile main loop.
//
// Orientation used everywhere: the MFMA "A" operand is a tile of the classifier C (vocabulary
// rows), the "B" operand a tile of the embeddings E (token rows), so a 32x32 accumulator block
// holds logits^T: lane l owns token (l % 32) and the 16 vocabulary rows
//     8 * (r / 4) + 4 * (l / 32) + (r % 4),  r = 0..15.
// A lane therefore sees many classes of ONE token, which makes the per-token soft-max
// statistics a register-local reduction.
#pragma once

#include <atomic>
#include <utility>

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cce_hip.h"

namespace cce {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr int kBK = 64;          // reduction elements per LDS stage
constexpr int kRowBytes = 128;   // kBK * sizeof(16-bit element)

struct BF16 {};
struct F16 {};

template <typename T>
struct Elem;

template <>
struct Elem<BF16> {
  using vec8 = bf16x8_t;
  static __device__ __forceinline__ float to_float(uint16_t bits) {
    return __uint_as_float(static_cast<uint32_t>(bits) << 16);
  }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    __bf16 h = static_cast<__bf16>(f);
    return __builtin_bit_cast(uint16_t, h);
  }
  // two floats -> one packed pair (lo in the low half), one conversion instruction
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef float float2_t __attribute__((ext_vector_type(2)));
    float2_t f;
    f[0] = lo;
    f[1] = hi;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
  }
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // 16 x 16 block, 32 reduction elements: lane l holds row (l % 16), elements 8 (l / 16) .. + 7 of either operand
  // and, of the result, column (l % 16), rows 4 (l / 16) + r, r = 0 .. 3.
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // The same MFMA with the accumulator pinned to one register file: "a" = the accumulation registers
  // (AGPRs), "v" = the ordinary ones.  For kernels whose accumulators outnumber the 256 AGPRs: the
  // compiler places the results of all MFMA builtins of a function in one file and spills the excess,
  // so such a kernel writes every one of its MFMAs this way.  The compiler cannot see the MFMA inside
  // the asm statement and inserts none of the wait states the matrix pipeline needs around register
  // copies it may place next to it, so the statement carries them itself: 5 before (an operand just
  // written by a move) and 12 after (the result of this 8-pass MFMA read by a move).  They hide under
  // the 32 cycles the MFMA occupies the pipeline anyway.
  static __device__ __forceinline__ void mfma_agpr(vec8 a, vec8 b, f32x16& c) {
    asm volatile("s_nop 4\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\ts_nop 11" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_vgpr(vec8 a, vec8 b, f32x16& c) {
    asm volatile("s_nop 4\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\ts_nop 11" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void atomic_add_pair(uint16_t* addr, float lo, float hi) {
    bf16x2_t v;
    v[0] = static_cast<__bf16>(lo);
    v[1] = static_cast<__bf16>(hi);
    __builtin_amdgcn_global_atomic_fadd_v2bf16(reinterpret_cast<bf16x2_t*>(addr), v);
  }
};

template <>
struct Elem<F16> {
  using vec8 = f16x8_t;
  static __device__ __forceinline__ float to_float(uint16_t bits) {
    return static_cast<float>(__builtin_bit_cast(_Float16, bits));
  }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    _Float16 h = static_cast<_Float16>(f);
    return __builtin_bit_cast(uint16_t, h);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef float float2_t __attribute__((ext_vector_type(2)));
    float2_t f;
    f[0] = lo;
    f[1] = hi;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2_t));
  }
  static __device__ __forceinline__ f32x16 mfma(vec8 a, vec8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ void mfma_agpr(vec8 a, vec8 b, f32x16& c) {
    asm volatile("s_nop 4\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\ts_nop 11" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_vgpr(vec8 a, vec8 b, f32x16& c) {
    asm volatile("s_nop 4\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\ts_nop 11" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void atomic_add_pair(uint16_t* addr, float lo, float hi) {
    f16x2_t v;
    v[0] = static_cast<_Float16>(lo);
    v[1] = static_cast<_Float16>(hi);
    __builtin_amdgcn_global_atomic_fadd_v2f16(reinterpret_cast<f16x2_t*>(addr), v);
  }
};

// The result of an MFMA written as inline assembly may be read by another kind of instruction only
// after the matrix pipeline has drained (up to 18 wait states for a 32 x 32 block); the compiler
// inserts those for its own MFMAs but cannot see into an asm statement.
__device__ __forceinline__ void mfma_drain(f32x16& c) { asm volatile("s_nop 15\n\ts_nop 3" : "+v"(c)); }
__device__ __forceinline__ void mfma_drain_all() { asm volatile("s_nop 15\n\ts_nop 3" ::: "memory"); }

// Constants of soft-capping in the log2 domain: for a raw logit x the kernels form
// s * log2(e) = out_scale * tanh(x / softcap) with tanh(u) = 1 - 2 / (1 + exp2(x * in_scale)).
struct Softcap {
  float in_scale;   // 2 * log2(e) / softcap
  float out_scale;  // softcap * log2(e)
  int on;
};

__host__ __device__ inline Softcap make_softcap(float softcap) {
  Softcap s;
  s.on = (softcap > 0.0f) ? 1 : 0;  // false for NaN as well
  s.in_scale = s.on ? 2.0f * kLog2e / softcap : 0.0f;
  s.out_scale = s.on ? softcap * kLog2e : 0.0f;
  return s;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Sum over the 16 lanes of a row (lanes 16 k .. 16 k + 15), left in every lane of the row: four rotations on the
// vector unit, no LDS crossbar.
__device__ __forceinline__ float row16_sum(float v) {
  auto ror = [](float x, auto ctrl) {
    const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, false);
    return __builtin_bit_cast(float, r);
  };
  using std::integral_constant;
  v += ror(v, integral_constant<int, 0x121>{});  // row_ror:1
  v += ror(v, integral_constant<int, 0x122>{});  // row_ror:2
  v += ror(v, integral_constant<int, 0x124>{});  // row_ror:4
  v += ror(v, integral_constant<int, 0x128>{});  // row_ror:8
  return v;
}

// Maximum over the 64 lanes as a wave-uniform value, on the vector unit alone: four rotations inside the rows of 16
// lanes (after which every lane holds its row's maximum), then lane 15 of rows 0 and 2 broadcast into rows 1 and 3
// and lane 31 into rows 2 and 3; the last lane then holds the maximum of all.  The shuffles of wave_max() above
// go through the LDS crossbar (one ds_bpermute and a wait each).
__device__ __forceinline__ float wave_max_uniform(float v) {
  auto dpp = [](float x, auto ctrl, auto row_mask) {
    const int r = __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), decltype(ctrl)::value,
                                              decltype(row_mask)::value, 0xf, false);
    return __builtin_bit_cast(float, r);
  };
  using std::integral_constant;
  v = fmaxf(v, dpp(v, integral_constant<int, 0x121>{}, integral_constant<int, 0xf>{}));  // row_ror:1
  v = fmaxf(v, dpp(v, integral_constant<int, 0x122>{}, integral_constant<int, 0xf>{}));  // row_ror:2
  v = fmaxf(v, dpp(v, integral_constant<int, 0x124>{}, integral_constant<int, 0xf>{}));  // row_ror:4
  v = fmaxf(v, dpp(v, integral_constant<int, 0x128>{}, integral_constant<int, 0xf>{}));  // row_ror:8
  v = fmaxf(v, dpp(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xa>{}));  // row_bcast:15 into rows 1, 3
  v = fmaxf(v, dpp(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xc>{}));  // row_bcast:31 into rows 2, 3
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fminf(v, __shfl_xor(v, off, 64));
  return v;
}

// ---------------------------------------------------------------------------------------------
// Global -> register -> LDS loader for ROWS rows of kBK 16-bit elements.
// LDS image: row-major, 128 bytes per row, the eight 16-byte chunks of a row XOR-swizzled with
// (row & 7) so that the 32 rows an MFMA operand fetch touches fall into distinct banks.
// Thread t owns chunk (t & 7) of rows (t / 8) + q * (NT / 8).
// ---------------------------------------------------------------------------------------------
template <int ROWS, int NT, bool ALIGNED>
struct RowLoader {
  static constexpr int NQ = ROWS * 8 / NT;
  static constexpr int ROWSTEP = NT / 8;
  static_assert(ROWS * 8 % NT == 0, "tile rows must divide evenly over the threads");
  static_assert(ROWSTEP % 8 == 0, "swizzle must not depend on q");

  const uint16_t* ptr[NQ];  // row base or nullptr for a row outside the matrix
  uint4 reg[NQ];

  // ALIGNED: rows are 16-byte aligned, unit element stride and D % 8 == 0.
  __device__ __forceinline__ void load(int k0, int D, int64_t stride_k) {
    const int k = k0 + (threadIdx.x & 7) * 8;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (ALIGNED) {
        if (ptr[q] != nullptr && k < D) v = *reinterpret_cast<const uint4*>(ptr[q] + k);
      } else {
        if (ptr[q] != nullptr) {
          uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            uint32_t x = (k + i < D) ? static_cast<uint32_t>(ptr[q][static_cast<int64_t>(k + i) * stride_k]) : 0u;
            w[i >> 1] |= x << ((i & 1) * 16);
          }
          v = make_uint4(w[0], w[1], w[2], w[3]);
        }
      }
      reg[q] = v;
    }
  }

  __device__ __forceinline__ void store(unsigned char* lds) const {
    const int row0 = threadIdx.x >> 3;
    const int chunk = (threadIdx.x & 7) ^ (row0 & 7);
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      *reinterpret_cast<uint4*>(lds + (row0 + q * ROWSTEP) * kRowBytes + (chunk << 4)) = reg[q];
    }
  }
};

// ---------------------------------------------------------------------------------------------
// One logit tile: acc[vi][ti] += C_tile (TILE_V x D) * E_tile^T (D x TILE_T), both streamed through
// two LDS stages of kBK columns.  Wave (wv, wt) of an NWV x NWT grid owns WV x WT accumulator
// blocks of 32 x 32.  `lds` must hold 2 * (TILE_V + TILE_T) * 128 bytes.  Ends with a barrier, so
// the LDS may be reused right after the call.
// ---------------------------------------------------------------------------------------------
template <typename T, int WV, int WT, int NWV, int NWT, bool ALIGNED>
struct LogitTile {
  static constexpr int TILE_V = 32 * WV * NWV;
  static constexpr int TILE_T = 32 * WT * NWT;
  static constexpr int NT = 64 * NWV * NWT;
  static constexpr int STAGE_BYTES = (TILE_V + TILE_T) * kRowBytes;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;

  using CLoader = RowLoader<TILE_V, NT, ALIGNED>;
  using ELoader = RowLoader<TILE_T, NT, ALIGNED>;

  static __device__ __forceinline__ void run(f32x16 (&acc)[WV][WT], CLoader& cl, ELoader& el,
                                             unsigned char* lds, int D, int64_t stride_ck) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wv = wave / NWT;
    const int wt = wave % NWT;
    const int l32 = lane & 31;
    const int half = lane >> 5;

#pragma unroll
    for (int vi = 0; vi < WV; ++vi)
#pragma unroll
      for (int ti = 0; ti < WT; ++ti)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[vi][ti][r] = 0.0f;

    const int nk = (D + kBK - 1) / kBK;
    cl.load(0, D, stride_ck);
    el.load(0, D, 1);
    cl.store(lds);
    el.store(lds + TILE_V * kRowBytes);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      unsigned char* cur = lds + (kt & 1) * STAGE_BYTES;
      unsigned char* nxt = lds + ((kt + 1) & 1) * STAGE_BYTES;
      const bool more = (kt + 1) < nk;
      if (more) {
        cl.load((kt + 1) * kBK, D, stride_ck);
        el.load((kt + 1) * kBK, D, 1);
      }
      const unsigned char* cbase = cur + (wv * WV * 32 + l32) * kRowBytes;
      const unsigned char* ebase = cur + (TILE_V + wt * WT * 32 + l32) * kRowBytes;
      const int sw = l32 & 7;
#pragma unroll
      for (int kk = 0; kk < kBK / 16; ++kk) {
        typename Elem<T>::vec8 a[WV], b[WT];
        const int coff = (((kk * 2 + half) ^ sw) << 4);
#pragma unroll
        for (int vi = 0; vi < WV; ++vi)
          a[vi] = __builtin_bit_cast(typename Elem<T>::vec8,
                                     *reinterpret_cast<const uint4*>(cbase + vi * 32 * kRowBytes + coff));
#pragma unroll
        for (int ti = 0; ti < WT; ++ti)
          b[ti] = __builtin_bit_cast(typename Elem<T>::vec8,
                                     *reinterpret_cast<const uint4*>(ebase + ti * 32 * kRowBytes + coff));
#pragma unroll
        for (int vi = 0; vi < WV; ++vi)
#pragma unroll
          for (int ti = 0; ti < WT; ++ti) acc[vi][ti] = Elem<T>::mfma(a[vi], b[ti], acc[vi][ti]);
      }
      if (more) {
        cl.store(nxt);
        el.store(nxt + TILE_V * kRowBytes);
      }
      __syncthreads();
    }
  }
};

// ---------------------------------------------------------------------------------------------
// Logit tile with direct global -> LDS loads (gfx950 `global_load_lds_dwordx4`): the data never
// passes through registers and no wave spends issue slots on LDS stores.
//
// Stage = 64 reduction columns = 128-byte rows, so that every row segment is one full cache line
// (measured: the L2 -> LDS path delivers ~16 TB/s with 128-byte segments, ~12 TB/s with 64-byte
// ones, and that path is as scarce as the MFMA time at this tile size).  One load writes 64 lanes x
// 16 bytes = 1 KB of contiguous LDS = 8 rows; lane l lands in row (l >> 3), chunk slot (l & 7) of its
// block and fetches global chunk slot ^ ((row >> 1) & 7), the XOR swizzle the fragment reads undo
// (16 consecutive rows x one chunk then cover all 64 banks).  Block b of a stage (b = q * NW + wave)
// holds rows [8 b, 8 b + 8): class rows first, then token rows.
//
// The loads are inline assembly (the compiler would otherwise wait for every outstanding load
// before the next LDS read) and completion is tracked by hand: two LDS stages, one barrier per stage
// placed before the last of the four 16-column steps.  At that barrier every wave has read its last
// fragments of stage s, so the loads of stage s + 2 may go into that LDS stage from there on; they are
// spread over the next two steps, and the first fragments of stage s + 1 are read under the MFMAs
// of the last step.
// ---------------------------------------------------------------------------------------------
// M0 (the LDS address of the load) is a reserved register; naming it in the clobber list is what tells the
// compiler that the statement changes it, and clang remarks on exactly that.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_dma16(const void* gptr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr)
               : "memory", "m0");
}
// The same with the address split into a wave-uniform 64-bit base (scalar registers) and a 32-bit byte offset per
// lane: half the vector registers per address, and what changes from stage to stage is added on the scalar unit.
__device__ __forceinline__ void lds_dma16_sbase(const void* sbase, unsigned voff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr)
               : "memory", "m0");
}
#pragma clang diagnostic pop

template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a compile-time constant
// in every iteration, whatever the size of its body (an array of accumulators indexed by it stays in registers).
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// s_waitcnt vmcnt(N) with a compile-time N
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

constexpr int kDmaBK = 64;
constexpr int kDmaRowBytes = 128;

template <typename T, int WV, int WT, int NWV, int NWT>
struct DmaLogitTile {
  static constexpr int TILE_V = 32 * WV * NWV;
  static constexpr int TILE_T = 32 * WT * NWT;
  static constexpr int NW = NWV * NWT;
  static constexpr int NT = 64 * NW;
  static constexpr int STAGE_BYTES = (TILE_V + TILE_T) * kDmaRowBytes;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static constexpr int NQC = TILE_V / 8 / NW;  // loads per wave and stage that fetch class rows
  static constexpr int NQE = TILE_T / 8 / NW;  // ... token rows
  static constexpr int NQ = NQC + NQE;
  // The loads of a stage are issued in two groups, one load after every second MFMA: [0, QA) under step 3
  // of the stage before last and [QA, NQ) under step 0 of the last, which leaves them steps 1 and 2 to land
  // (measured: 1 % faster than three groups over steps 3, 0 and 1 with one step to land).
  static constexpr int QA = (NQ + 1) / 2;
  static constexpr int QB = NQ;
  static_assert(TILE_V % (8 * NW) == 0 && TILE_T % (8 * NW) == 0, "blocks must divide over the waves");
  static_assert(NW % 2 == 0, "the swizzle of a lane must not depend on q");
  using vec8 = typename Elem<T>::vec8;

  // Tile row (class or token index inside the tile) that this lane fetches with load q.
  static __device__ __forceinline__ int row_of(int q, int wave, int lane) {
    const int q2 = (q < NQC) ? q : q - NQC;
    return 8 * (q2 * NW + wave) + (lane >> 3);
  }
  // Element offset inside a 64-column stage of the chunk this lane fetches.
  static __device__ __forceinline__ int chunk_elems(int wave, int lane) {
    const int sw = (4 * (wave & 1) + (lane >> 4)) & 7;  // (row >> 1) & 7 for row = 8 * block + (lane >> 3)
    return ((lane & 7) ^ sw) * 8;
  }

  struct Frags {
    vec8 a[WV];
    vec8 b[WT];
  };

  static __device__ __forceinline__ Frags read_frags(const unsigned char* lds, int stage_off, int kk, int coff0,
                                                     int eoff0, int sw, int half) {
    Frags f;
    const int chunk = (((kk * 2 + half) ^ sw) << 4);
    const unsigned char* cb = lds + stage_off + coff0 + chunk;
    const unsigned char* eb = lds + stage_off + eoff0 + chunk;
#pragma unroll
    for (int vi = 0; vi < WV; ++vi)
      f.a[vi] = __builtin_bit_cast(vec8, *reinterpret_cast<const uint4*>(cb + vi * 32 * kDmaRowBytes));
#pragma unroll
    for (int ti = 0; ti < WT; ++ti)
      f.b[ti] = __builtin_bit_cast(vec8, *reinterpret_cast<const uint4*>(eb + ti * 32 * kDmaRowBytes));
    return f;
  }

  // Issue load q of one stage (columns [k0, k0 + 64)) into LDS stage `stage_off`.
  static __device__ __forceinline__ void issue_one(const uint16_t* const (&ptr)[NQ], int q, int k0, unsigned lds_base,
                                                   int stage_off, int wave) {
    const int blk = (q < NQC) ? (q * NW + wave) : (TILE_V / 8 + (q - NQC) * NW + wave);
    lds_dma16(ptr[q] + k0, lds_base + stage_off + blk * 1024);
  }

  // One 16-column step: the MFMAs on fragment set `cur`, and between them (one memory instruction per
  // MFMA, so that this wave alone keeps the matrix pipeline fed while it issues them)
  //   * the LDS reads of the next set `nxt` (step rkk of LDS stage rstage), ordered as the next step's
  //     MFMAs will want them, and
  //   * the direct-to-LDS loads [Q0, Q1) of a later stage, one after every second MFMA.
  // Measured: a burst of all the loads of a stage right after the barrier backs up the address path,
  // the waves that issue last fall a third of a stage behind and everybody waits for them at the next
  // barrier; and a burst of fragment reads at the top of a step idles the matrix pipeline whenever both
  // waves of a SIMD are in that burst together, which the barriers make the rule.
  template <int Q0, int Q1>
  static __device__ __forceinline__ void step(f32x16 (&acc)[WV][WT], const Frags& cur, Frags& nxt,
                                              const unsigned char* lds, int rstage, int rkk, int coff0, int eoff0,
                                              int sw, int half, const uint16_t* const (&ptr)[NQ], int k0,
                                              unsigned lds_base, int lstage, int wave) {
    static_assert(Q1 - Q0 <= (WV * WT) / 2, "one load per two MFMAs");
    static_assert(WV + WT <= WV * WT, "one fragment read per MFMA");
    const int chunk = (((rkk * 2 + half) ^ sw) << 4);
    const unsigned char* cb = lds + rstage + coff0 + chunk;
    const unsigned char* eb = lds + rstage + eoff0 + chunk;
#pragma unroll
    for (int vi = 0; vi < WV; ++vi)
#pragma unroll
      for (int ti = 0; ti < WT; ++ti) {
        acc[vi][ti] = Elem<T>::mfma(cur.a[vi], cur.b[ti], acc[vi][ti]);
        const int idx = vi * WT + ti;
        __builtin_amdgcn_sched_barrier(0);
        if (idx == 0) {
          nxt.a[0] = __builtin_bit_cast(vec8, *reinterpret_cast<const uint4*>(cb));
        } else if (idx <= WT) {
          nxt.b[idx - 1] = __builtin_bit_cast(vec8, *reinterpret_cast<const uint4*>(eb + (idx - 1) * 32 * kDmaRowBytes));
        } else if (idx < WV + WT) {
          nxt.a[idx - WT] = __builtin_bit_cast(vec8, *reinterpret_cast<const uint4*>(cb + (idx - WT) * 32 * kDmaRowBytes));
        }
        if ((idx & 1) && Q0 + idx / 2 < Q1) issue_one(ptr, Q0 + idx / 2, k0, lds_base, lstage, wave);
        __builtin_amdgcn_sched_barrier(0);
      }
  }

  // Start fetching a tile into the (idle) LDS ring: all of stage 0 and the first group of stage 1.
  // Called before the epilogue of the previous tile, so that the next main loop starts with data in LDS.
  static __device__ __forceinline__ void prefetch(const uint16_t* const (&ptr)[NQ], unsigned char* lds, int D) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));
    const int last = (D / kDmaBK - 1) * kDmaBK;
#pragma unroll
    for (int q = 0; q < NQ; ++q) issue_one(ptr, q, 0, lds_base, 0, wave);
#pragma unroll
    for (int q = 0; q < QA; ++q) issue_one(ptr, q, min(kDmaBK, last), lds_base, STAGE_BYTES, wave);
  }

  // D must be a multiple of 64.  prefetch() with the same pointers must have been called, and nothing
  // may have touched the LDS ring since.
  static __device__ __forceinline__ void run(f32x16 (&acc)[WV][WT], const uint16_t* const (&ptr)[NQ],
                                             unsigned char* lds, int D) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wv = wave / NWT;
    const int wt = wave % NWT;
    const int l32 = lane & 31;
    const int half = lane >> 5;
    const int sw = (l32 >> 1) & 7;
    const int coff0 = (wv * WV * 32 + l32) * kDmaRowBytes;
    const int eoff0 = (TILE_V + wt * WT * 32 + l32) * kDmaRowBytes;
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));

#pragma unroll
    for (int vi = 0; vi < WV; ++vi)
#pragma unroll
      for (int ti = 0; ti < WT; ++ti)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[vi][ti][r] = 0.0f;

    const int nk = D / kDmaBK;
    const int last = (nk - 1) * kDmaBK;
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(QA) : "memory");  // stage 0 landed, stage 1 may be in flight
    __syncthreads();
    Frags fa = read_frags(lds, 0, 0, coff0, eoff0, sw, half);
    Frags fb;

    // The scheduling fences inside step() pin the interleaving: left alone, the compiler sinks every
    // LDS read next to its use and the LDS latency is exposed.
#pragma unroll 1
    for (int s = 0; s < nk; ++s) {
      const int cur = (s & 1) * STAGE_BYTES;
      const int nxt = STAGE_BYTES - cur;
      const int k1 = min((s + 1) * kDmaBK, last);
      const int k2 = min((s + 2) * kDmaBK, last);
      step<QA, QB>(acc, fa, fb, lds, cur, 1, coff0, eoff0, sw, half, ptr, k1, lds_base, nxt, wave);  // step 0
      step<QB, NQ>(acc, fb, fa, lds, cur, 2, coff0, eoff0, sw, half, ptr, k1, lds_base, nxt, wave);  // step 1
      step<NQ, NQ>(acc, fa, fb, lds, cur, 3, coff0, eoff0, sw, half, ptr, k1, lds_base, nxt, wave);  // step 2
      // Stage s + 1 (last loads issued under step 0) has landed for this wave; after the barrier, for
      // every wave, and every wave holds its last fragments of stage s in registers: that LDS stage is
      // free and the first loads of stage s + 2 go into it.  A prefetch past the end re-reads the last
      // stage (never consumed), which keeps the loop free of branches.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      step<0, QA>(acc, fb, fa, lds, nxt, 0, coff0, eoff0, sw, half, ptr, k2, lds_base, cur, wave);  // step 3
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the last, unused prefetch
    __syncthreads();  // every wave is done with the LDS (the last prefetch was awaited above)
  }
};

// ---------------------------------------------------------------------------------------------
// The same logit tile from 16 x 16 x 32 MFMAs.  The matrix pipes of this chip are limited by power, not by
// issue: with operands of full entropy the 32 x 32 x 16 instruction sustains 1.84 PFLOP/s from registers alone
// and the 16 x 16 x 32 one 2.09 (it reads and writes a quarter of the accumulator registers per instruction and
// adds twice as many products before it touches them), both 2.46 with operands of zeros; the clock the chip holds
// under the forward kernel rises accordingly.  Same tile, ring and loads as DmaLogitTile; what changes is who
// holds what:
//   wave (wv, wt) owns WV x WT blocks of 16 classes x 16 token rows; lane l holds, of every block, the token row
//   (l % 16) and the classes 4 (l / 16) + r, r = 0 .. 3; a fragment is 16 rows x 32 reduction columns = half a
//   ring row, lane l reads 16-byte chunk (l / 16) (+ 4 for the second half) of row (l % 16): one fragment read is
//   four groups of 16 rows x one chunk, each covering all 64 banks through the XOR swizzle.
// Pipeline, per 64-column stage two steps of WV x WT MFMAs: the step on columns 0 .. 31 reads the fragments of
// columns 32 .. 63 of the same stage, the step on columns 32 .. 63 those of the next stage's first half and
// issues ALL loads of the stage after that into the ring stage it has just finished with.  A class fragment
// is re-read in place as soon as its WT MFMAs are issued (so only the token fragments are held twice); one
// barrier per stage, a few MFMAs into the second step, at which the loads issued most of a stage earlier have landed.
// The stages run on across the tiles of a span: the loads issued under the last two stages of a tile fetch the
// first two stages of the NEXT tile (next_tile() swaps the class pointers), so that nothing is fetched that is
// not consumed and the next main loop starts with its data in LDS, whatever the epilogue in between does.
// `buf` carries the ring stage the next tile starts in (it alternates when D / 64 is odd).
// ---------------------------------------------------------------------------------------------
template <typename T, int WV, int WT, int NWV, int NWT>
struct DmaLogitTile16 {
  static_assert(WV % 2 == 0 && WT % 2 == 0, "the ring is addressed in blocks of 32 rows");
  using Base = DmaLogitTile<T, WV / 2, WT / 2, NWV, NWT>;
  static constexpr int TILE_V = Base::TILE_V;
  static constexpr int TILE_T = Base::TILE_T;
  static constexpr int NW = Base::NW;
  static constexpr int STAGE_BYTES = Base::STAGE_BYTES;
  static constexpr int LDS_BYTES = Base::LDS_BYTES;
  static constexpr int NQC = Base::NQC;
  static constexpr int NQ = Base::NQ;
  using vec8 = typename Elem<T>::vec8;

  static __device__ __forceinline__ int row_of(int q, int wave, int lane) { return Base::row_of(q, wave, lane); }
  static __device__ __forceinline__ int chunk_elems(int wave, int lane) { return Base::chunk_elems(wave, lane); }

  // Where the loads of a tile come from.  A load fetches 8 rows x 128 bytes; its address is a wave-uniform 64-bit base
  // (scalar registers) plus a 32-bit byte offset per lane.  Token rows are gathered, so each of their loads has an
  // offset of its own relative to the matrix (e_off).  Class rows are consecutive: the base of load q is the first
  // row of its block of 8 and the lane adds (its row in the block) x (row stride) + (its chunk); for a tile that
  // reaches past the last class the block is moved back inside and the row clamped to c_lim[q], so that every
  // lane reads a row that exists (what it feeds is masked in the epilogue).  Only c_blk / c_lim change from tile
  // to tile, on the scalar unit.
  struct Source {
    unsigned e_off[NQ - NQC];
    const unsigned char* e_base;
    const unsigned char* c_blk[NQC];
    int c_lim[NQC];
    unsigned c_stride_bytes;
    unsigned row_in_block;  // lane >> 3
    unsigned chunk_bytes;   // byte offset of this lane's 16-byte chunk inside a 128-byte row segment
  };

  // Points the class loads of `src` at the tile whose first class row is `tile` and which has `left` >= 1 classes
  // inside the matrix (256 or more: a whole tile).
  static __device__ __forceinline__ void set_class_tile(Source& src, const unsigned char* tile, int left, int wave) {
#pragma unroll
    for (int q = 0; q < NQC; ++q) {
      const int first = 8 * (q * NW + wave);
      const int blk = min(first, left - 1);
      src.c_blk[q] = tile + static_cast<int64_t>(blk) * src.c_stride_bytes;
      src.c_lim[q] = left - 1 - blk;
    }
  }

  static __device__ __forceinline__ vec8 frag(const unsigned char* p) {
    return __builtin_bit_cast(vec8, *reinterpret_cast<const uint4*>(p));
  }

  // Load q of one stage, columns [k0, k0 + 64), into ring stage `stage_off`.
  static __device__ __forceinline__ void issue_one(const Source& src, int q, int k0, unsigned lds_base, int stage_off,
                                                   int wave) {
    if (q < NQC) {
      const unsigned row = min(src.row_in_block, static_cast<unsigned>(src.c_lim[q]));
      lds_dma16_sbase(src.c_blk[q] + 2 * k0, row * src.c_stride_bytes + src.chunk_bytes,
                      lds_base + stage_off + (q * NW + wave) * 1024);
    } else {
      lds_dma16_sbase(src.e_base + 2 * k0, src.e_off[q - NQC],
                      lds_base + stage_off + (TILE_V / 8 + (q - NQC) * NW + wave) * 1024);
    }
  }

  // One step: WV x WT MFMAs on the class fragments a[] and the token fragments bc[]; under them, at most one
  // memory instruction after each MFMA:
  //   READ  the fragments of the next step from rd_c / rd_e (ring stage + this lane's chunk): class fragment vi
  //         into a[vi] once the last MFMA that uses the old one is issued, the token fragments into bn[];
  //   LOAD  all loads of a later stage (columns koff ..) into ring stage `ld_stage`.
  // SYNC (the step on the second half of a stage): after the first WT MFMAs, which need nothing new, this wave
  // waits for its own loads of the next stage and for the fragment reads it still has in flight, then the
  // barrier: from there on the next stage may be read and the stage this step computes on (every wave holds
  // its last fragments of it) may be overwritten.  Reads and loads of such a step all come after the barrier.
  // (With the barrier between the steps instead, every wave met it with its last fragment read just issued and
  // the compute units idled a sixth of the time.)
  static constexpr int kSyncAt = WT;  // MFMAs of a SYNC step issued before the barrier
  static constexpr int kSlots = WV * WT;
  static constexpr int a_slot(bool sync, int vi) {
    const int natural = vi * WT + WT - 1;  // the last MFMA that reads a[vi]
    return (sync && natural < kSyncAt + 1 + 2 * vi) ? kSyncAt + 1 + 2 * vi : natural;
  }
  static constexpr int b_slot(bool sync, int t) {
    return sync ? kSyncAt + 5 + t * ((kSlots - kSyncAt - 8) / WT & ~1) : 1 + t * (kSlots / WT);
  }
  static constexpr int load_slot(int j) { return j < 6 ? kSyncAt + 2 + 4 * j : kSlots - 4 + 2 * (j - 6); }
  static_assert(WV == 8 && WT == 4 && NQ == 8, "the slot tables above are laid out for 8 x 4 blocks and 8 loads");

  // ZERO (the first step of a tile): the accumulators start from the instruction's constant zero instead of being
  // cleared beforehand (128 register writes per lane and tile; the copy of the first stage this takes costs a
  // cool chip with idle operands 3 %, and gains 2 % under real operands, where the chip is power-bound).
  template <bool READ, bool LOAD, bool SYNC, bool ZERO = false>
  static __device__ __forceinline__ void step(f32x4 (&acc)[WV][WT], vec8 (&a)[WV], const vec8 (&bc)[WT], vec8 (&bn)[WT],
                                              const unsigned char* rd_c, const unsigned char* rd_e, const Source& src,
                                              int koff, unsigned lds_base, int ld_stage, int wave) {
    static_for<WV * WT>([&](auto idx_c) {
      constexpr int idx = decltype(idx_c)::value;
      constexpr int vi = idx / WT, ti = idx % WT;
      if (SYNC && idx == kSyncAt) {
        wait_vmcnt<0>();
        __syncthreads();
      }
      acc[vi][ti] = Elem<T>::mfma16(a[vi], bc[ti], ZERO ? f32x4{0.0f, 0.0f, 0.0f, 0.0f} : acc[vi][ti]);
      __builtin_amdgcn_sched_barrier(0);
      if (READ) {
        static_for<WT>([&](auto t_c) {
          constexpr int t = decltype(t_c)::value;
          if (idx == b_slot(SYNC, t)) bn[t] = frag(rd_e + t * 16 * kDmaRowBytes);
        });
        static_for<WV>([&](auto v_c) {
          constexpr int v = decltype(v_c)::value;
          if (idx == a_slot(SYNC, v)) a[v] = frag(rd_c + v * 16 * kDmaRowBytes);
        });
      }
      if (LOAD) {
        static_for<NQ>([&](auto j_c) {
          constexpr int j = decltype(j_c)::value;
          if (idx == load_slot(j)) issue_one(src, j, koff, lds_base, ld_stage, wave);
        });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  }

  // Start the ring for the first tile of a span: its first two stages, into ring stages 0 and 1.
  static __device__ __forceinline__ void prefetch(const Source& src, unsigned char* lds) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));
#pragma unroll
    for (int q = 0; q < NQ; ++q) issue_one(src, q, 0, lds_base, 0, wave);
#pragma unroll
    for (int q = 0; q < NQ; ++q) issue_one(src, q, kDmaBK, lds_base, STAGE_BYTES, wave);
  }

  // D must be a multiple of 64 and at least 128.  The first two stages of this tile must be in flight or landed in
  // ring stages buf, 1 - buf (prefetch() for the first tile of a span: first_tile; else the previous run()), and
  // nothing else may have touched the ring.
  // next_tile() is called once, when the class rows of this tile have been fetched for the last time: it points
  // `src` at the tile whose first stages the rest of this run fetches (or leaves it: those loads then repeat this
  // tile's first stages and are never read).
  template <typename NextTile>
  static __device__ __forceinline__ void run(f32x4 (&acc)[WV][WT], Source& src, unsigned char* lds, int D, int& buf,
                                             bool first_tile, NextTile&& next_tile) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wv = wave / NWT;
    const int wt = wave % NWT;
    const int r16 = lane & 15;
    // this lane's 16-byte chunk of a ring row: (l / 16) for the first half of a stage, + 4 for the second,
    // XOR-swizzled with (row >> 1) & 7 like the loads place them
    const int chunk0 = (((lane >> 4) ^ (r16 >> 1)) << 4);
    const int chunk1 = chunk0 ^ 64;
    const unsigned char* c_row = lds + (wv * WV * 16 + r16) * kDmaRowBytes;
    const unsigned char* e_row = lds + (TILE_V + wt * WT * 16 + r16) * kDmaRowBytes;
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));

    const int nk = D / kDmaBK;
    int cur = buf * STAGE_BYTES;
    if (first_tile) {
      wait_vmcnt<NQ>();  // the first stage has landed for this wave (the second may be in flight) ...
      __syncthreads();   // ... and for all of them
    }
    // (a later tile's first stage was awaited by every wave before the last barrier of the tile before it: no
    // barrier here, so a wave that leaves its epilogue early starts on the next tile while the others finish)
    vec8 a[WV], b0[WT], b1[WT];
#pragma unroll
    for (int ti = 0; ti < WT; ++ti) b0[ti] = frag(e_row + cur + chunk0 + ti * 16 * kDmaRowBytes);
#pragma unroll
    for (int vi = 0; vi < WV; ++vi) a[vi] = frag(c_row + cur + chunk0 + vi * 16 * kDmaRowBytes);

    // first stage (never the last: D >= 128)
    {
      const int nxt = STAGE_BYTES - cur;
      step<true, false, false, true>(acc, a, b0, b1, c_row + cur + chunk1, e_row + cur + chunk1, src, 0, lds_base, 0, wave);
      if (nk == 2) next_tile();
      step<true, true, true>(acc, a, b1, b0, c_row + nxt + chunk0, e_row + nxt + chunk0, src, (2 < nk) ? 2 * kDmaBK : 0,
                             lds_base, cur, wave);
      cur = nxt;
    }
#pragma unroll 1
    for (int s = 1; s < nk - 1; ++s) {
      const int nxt = STAGE_BYTES - cur;
      step<true, false, false>(acc, a, b0, b1, c_row + cur + chunk1, e_row + cur + chunk1, src, 0, lds_base, 0, wave);
      if (s == nk - 2) next_tile();
      const int koff = (s + 2 < nk) ? (s + 2) * kDmaBK : 0;
      step<true, true, true>(acc, a, b1, b0, c_row + nxt + chunk0, e_row + nxt + chunk0, src, koff, lds_base, cur, wave);
      cur = nxt;
    }
    // the last stage: its second step reads nothing (the next tile's first fragments would sit in registers
    // through the epilogue) and fetches the second stage of the next tile
    step<true, false, false>(acc, a, b0, b1, c_row + cur + chunk1, e_row + cur + chunk1, src, 0, lds_base, 0, wave);
    step<false, true, true>(acc, a, b1, b0, c_row, e_row, src, kDmaBK, lds_base, cur, wave);
    buf = 1 - cur / STAGE_BYTES;
  }
};

inline int status_from_hip(hipError_t e) { return e == hipSuccess ? CCE_OK : static_cast<int>(e); }

// The dynamic LDS limit of a kernel (hipFuncAttributeMaxDynamicSharedMemorySize), set once per kernel and device
// instead of with every launch: it is a driver call, and the unfiltered backward launches dozens of kernels per
// step.  One object per kernel, a static at its launch site.
struct LdsLimitOnce {
  std::atomic<uint64_t> done{0};  // one bit per device
  template <typename K>
  hipError_t set(K kern, int bytes) {
    int dev = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return err;
    const uint64_t bit = uint64_t(1) << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (err == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return err;
  }
};

// Compute units of the current device (256 on an MI355X), looked up once per device.
inline int compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  int n = cached[dev & 63].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev & 63].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Vocabulary spans per row block for the kernels that cut the (row block, vocabulary) plane into
// items of one row block x one span of tiles.  Two things are weighed: the rounds of 256 workgroups
// the items make, and the L2 traffic of the 32 workgroups that run on one XCD at a time, which cover
// 32 / s row blocks (one E block each) times s spans (one stream of C tiles each): s + 32 / s streams,
// least for s = 4 .. 8.  The weight 0.165 is fitted to measurements at E [65536, 3584] x C [152064, 3584]
// (1, 2, 4, 8, 16 spans: 70.8, 62.5, 53.9, 56.8, 59.4 ms).
inline int choose_span_count(int nrb, int nvt) {
  const int num_cu = compute_units();  // (the size query and the launch must see the same device)
  int best = 1;
  double best_cost = 1e300;
  const int max_split = nvt < 64 ? nvt : 64;
  for (int s = 1; s <= max_split; ++s) {
    const int64_t items = static_cast<int64_t>(nrb) * s;
    const int64_t rounds = (items + num_cu - 1) / num_cu;
    const int tiles_per_item = (nvt + s - 1) / s;
    const double streams = (s <= 32) ? s + 32.0 / s : s + 1.0;
    const double traffic = 1.0 + 0.165 * (streams / 11.3137 - 1.0);
    const double cost = static_cast<double>(rounds) * tiles_per_item * traffic + 0.02 * s;
    if (cost < best_cost - 1e-9) {
      best_cost = cost;
      best = s;
    }
  }
  return best;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace cce
