// cce_backward_dz: the gradient of the loss with respect to the logits of one vocabulary chunk,
//     dz[i, j] = (p_ij (g_i + h_i) - [j == target_i] g_i) (1 - tanh^2)      p_ij = exp(s_ij - lse_i)
// written to memory in the input type (or as fp32), for the unfiltered ("exact") backward: with every entry of
// the gradient in play the two products dE = dz . C and dC = dz^T . E are dense matrix products over the chunk,
// which the kernels of cce_backward_dense.hip run.  The kernel is the forward kernel with another epilogue: same work
// items, same direct-to-LDS main loop, logits never leave the registers; only dz does, as row pieces of 128
// contiguous bytes (8 rows per wave instruction) after a transposition through LDS, while the first stages of the
// next tile are already arriving.
#include <type_traits>

#include "cce_dense.h"

namespace cce {

struct DzParams {
  const uint16_t* e;
  const uint16_t* c;
  const uint16_t* bias;
  const int32_t* valids;
  const float* lse;
  const float* d_out;
  const float* d_lse;
  const int64_t* targets;
  void* dz;
  int64_t ldz;
  int64_t n_rows, b, v, d;
  int64_t stride_e, stride_cv;
  int64_t shift, target_offset;
  float grad_scale;
  int d_out_is_scalar;
  int pad_store;  // also store the (zero) gradients of the classes between v and the end of their 16-byte piece,
                  // up to column ldz: the product kernels read dz in whole 64-class stages
  int nrb, nvt, nsplit, nitems, items_per_xcd;
  Softcap sc;
};

constexpr int kDzWV = 4, kDzWT = 2, kDzNWV = 2, kDzNWT = 4;  // the forward kernel's wave tiling
constexpr int kDzThreads = 64 * kDzNWV * kDzNWT;
constexpr int kDzTile = 256;
constexpr int kDzStageRow = 128;                  // bytes of one row of a wave's staged block (64 x 16-bit or 32 x fp32)
constexpr int kDzStageBytes = 32 * kDzStageRow;   // 32 rows

// OUT32: dz leaves as fp32 (for inputs that are fp32 values split into 16-bit parts along D, whose
// gradients are wanted at fp32 accuracy): a staged block is then 32 rows x 32 classes.
template <typename T, bool GENERAL, bool OUT32>
__global__ __launch_bounds__(kDzThreads, 1) void dense_dz_kernel(DzParams p) {
  using Fast = DmaLogitTile<T, kDzWV, kDzWT, kDzNWV, kDzNWT>;
  static_assert(kDzStageBytes * kDzNWV * kDzNWT <= Fast::TILE_T * kDmaRowBytes, "the staging blocks fit the token half of a stage");
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_addend = reinterpret_cast<float*>(smem + Fast::LDS_BYTES);  // [2][256]

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
  const int wv = wave / kDzNWT;
  const int wt = wave % kDzNWT;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int64_t t0 = static_cast<int64_t>(rb) * kDzTile;

  const uint16_t* fptr[Fast::NQ];
#pragma unroll
  for (int q = Fast::NQC; q < Fast::NQ; ++q) {
    int64_t i = t0 + Fast::row_of(q, wave, lane);
    i = (i < p.b) ? i : p.b - 1;  // rows past the end repeat the last one; their results are dropped
    const int64_t row = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
    fptr[q] = p.e + row * p.stride_e + Fast::chunk_elems(wave, lane);
  }

  // The two rows of this lane (one per 32-row column block): fixed for the whole item.
  float r_lse2[kDzWT], r_g[kDzWT], r_h[kDzWT];
  int r_tgt[kDzWT];
#pragma unroll
  for (int ti = 0; ti < kDzWT; ++ti) {
    const int64_t i = t0 + wt * (32 * kDzWT) + ti * 32 + l32;
    float lse2 = INFINITY, g = 0.0f, h = 0.0f;
    int tgt = -1;
    if (i < p.b) {
      const int64_t row = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
      lse2 = p.lse[i] * kLog2e;
      const int64_t tpos = row + p.shift;
      if (tpos < p.n_rows) {
        const int64_t t = p.targets[tpos] - p.target_offset;
        if (t >= 0 && t < p.v) tgt = static_cast<int>(t);
        g = p.grad_scale * (p.d_out_is_scalar ? p.d_out[0] : p.d_out[tpos]);
        if (p.d_lse != nullptr) h = p.d_lse[tpos];
      }
    }
    r_lse2[ti] = lse2;
    r_g[ti] = g;
    r_h[ti] = h;
    r_tgt[ti] = tgt;
  }

  // Staged blocks live in the token half of LDS stage 1, the one part of the ring that the early fetch of the
  // next tile (all of stage 0, the class half of stage 1) leaves alone.
  unsigned char* stage = smem + Fast::STAGE_BYTES + Fast::TILE_V * kDmaRowBytes + wave * kDzStageBytes;

  auto point_at_tile = [&](int vt) {
    const int64_t v0 = static_cast<int64_t>(vt) * kDzTile;
#pragma unroll
    for (int q = 0; q < Fast::NQC; ++q) {
      int64_t vr = v0 + Fast::row_of(q, wave, lane);
      vr = (vr < p.v) ? vr : p.v - 1;  // classes past the end repeat the last one; masked below
      fptr[q] = p.c + vr * p.stride_cv + Fast::chunk_elems(wave, lane);
    }
  };
  if (vt_begin < vt_end) {
    point_at_tile(vt_begin);
    Fast::prefetch(fptr, smem, static_cast<int>(p.d));
  }

  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int64_t v0 = static_cast<int64_t>(vt) * kDzTile;
    float* addend = s_addend + (vt & 1) * kDzTile;
    if (GENERAL) {
      if (tid < kDzTile) {  // published by the barriers of the main loop
        const int64_t vg = v0 + tid;
        float a = -INFINITY;
        if (vg < p.v) a = (p.bias != nullptr) ? Elem<T>::to_float(p.bias[vg]) : 0.0f;
        addend[tid] = a;
      }
    }
    f32x16 acc[kDzWV][kDzWT];
    Fast::run(acc, fptr, smem, static_cast<int>(p.d));  // (ends with a barrier: the ring is idle)
    // The next tile starts to arrive while this one's gradients are formed and stored.  Its loads sit ahead of the
    // stores below in the queue the main loop counts by: loads complete in order among themselves, so "at most QA
    // operations outstanding" at the top of run() still means that stage 0 has landed.
    if (vt + 1 < vt_end) {
      point_at_tile(vt + 1);
      Fast::prefetch(fptr, smem, static_cast<int>(p.d));
    }

    const int cls0 = static_cast<int>(v0) + wv * (32 * kDzWV);  // first class of this wave
    const float* wave_addend = addend + wv * (32 * kDzWV);
    const int sw = (l32 >> 1) & 7;  // 16-byte chunks of a staged row are XOR-swizzled with (row >> 1) & 7
#pragma unroll
    for (int ti = 0; ti < kDzWT; ++ti) {
      const float lse2 = r_lse2[ti], g = r_g[ti], gh = r_g[ti] + r_h[ti];
      const int tgt = r_tgt[ti];
      constexpr int kEs = OUT32 ? 4 : 2;                    // bytes per stored element
      constexpr int kViPer = kDzStageRow / (32 * kEs);      // 32-class blocks per staged block (2, or 1 for fp32)
      constexpr int kParts = kDzWV / kViPer;                // staged blocks per column block
      constexpr int kPieceElems = 16 / kEs;                 // elements per 16-byte piece
#pragma unroll
      for (int vh = 0; vh < kParts; ++vh) {
        // The gradients of one staged block.  One copy of the arithmetic per answer to "soft-capped?": asked per
        // logit, the (uniform) question costs two branches per element, a third of the epilogue's time.
        auto stage_block = [&](auto capped) {
#pragma unroll
          for (int vj = 0; vj < kViPer; ++vj) {
            const int vi = vh * kViPer + vj;
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
              float dzv[4];
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const int cl = vi * 32 + 8 * r4 + 4 * half + i;
                float x = acc[vi][ti][r4 * 4 + i];
                bool dead = false;
                if (GENERAL) {
                  const float add = wave_addend[cl];
                  dead = (add == -INFINITY);
                  x = dead ? 0.0f : x + add;
                }
                float s2, damp = 1.0f;
                if (decltype(capped)::value) {
                  const float t = __builtin_amdgcn_exp2f(x * p.sc.in_scale);
                  const float w = __builtin_amdgcn_rcpf(1.0f + t);
                  const float th = 1.0f - 2.0f * w;
                  s2 = p.sc.out_scale * th;
                  damp = 1.0f - th * th;
                } else {
                  s2 = x * kLog2e;
                }
                const float pr = __builtin_amdgcn_exp2f(s2 - lse2);
                float dz = pr * gh - ((cls0 + cl == tgt) ? g : 0.0f);
                if (decltype(capped)::value) dz *= damp;
                dzv[i] = dead ? 0.0f : dz;
              }
              const int col = (vj * 32 + 8 * r4 + 4 * half) * kEs;  // byte inside the staged row
              unsigned char* dst = stage + l32 * kDzStageRow + ((((col >> 4) ^ sw) << 4) | (col & 15));
              if (OUT32) {
                *reinterpret_cast<float4*>(dst) = make_float4(dzv[0], dzv[1], dzv[2], dzv[3]);
              } else {
                uint2 pk;
                pk.x = Elem<T>::pack2(dzv[0], dzv[1]);
                pk.y = Elem<T>::pack2(dzv[2], dzv[3]);
                *reinterpret_cast<uint2*>(dst) = pk;
              }
            }
          }
        };
        if (p.sc.on) {
          stage_block(std::true_type{});
        } else {
          stage_block(std::false_type{});
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the block is private to this wave: no barrier
        // 32 rows x 128 bytes leave as 16-byte pieces: one instruction covers 8 rows of 128 contiguous bytes
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int j = lane + 64 * k;
          const int row = j >> 3;
          const int pc = j & 7;
          const uint4 val = *reinterpret_cast<const uint4*>(stage + row * kDzStageRow + ((pc ^ ((row >> 1) & 7)) << 4));
          const int64_t gi = t0 + wt * (32 * kDzWT) + ti * 32 + row;
          const int64_t gcol = static_cast<int64_t>(cls0) + vh * (32 * kViPer) + pc * kPieceElems;
          if (gi < p.b) {
            unsigned char* dst = static_cast<unsigned char*>(p.dz) + (gi * p.ldz + gcol) * kEs;
            if (!GENERAL || gcol + kPieceElems <= p.v || (p.pad_store && gcol + kPieceElems <= p.ldz)) {
              *reinterpret_cast<uint4*>(dst) = val;
            } else if (OUT32) {
              const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (gcol + i < p.v) reinterpret_cast<uint32_t*>(dst)[i] = w[i];
            } else {
              const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
              for (int i = 0; i < 8; ++i)
                if (gcol + i < p.v) reinterpret_cast<uint16_t*>(dst)[i] = static_cast<uint16_t>(w[i >> 1] >> ((i & 1) * 16));
            }
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // reads done before the next block is staged
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The same kernel on the 16 x 16 x 32 main loop (DmaLogitTile16).  A lane holds, per 16-row block ti of its wave,
// ONE token row (lane % 16) and the classes 16 vi + 4 (lane / 16) + r of the wave's 128; what a row needs (its
// log-sum-exp, upstream gradients, target) sits in LDS, one entry per row of the workgroup, instead of in
// registers.  The whole ring is busy during the epilogue (the main loop fetches both first stages of the next
// tile under its last two stages), so the staging blocks have LDS of their own: 16 rows x 128 bytes per wave,
// half the classes of a row block at a time.
// ---------------------------------------------------------------------------------------------
constexpr int kDz16WV = 8, kDz16WT = 4;
constexpr int kDz16StageBytes = 16 * kDzStageRow;  // 16 rows of 128 bytes per wave

struct DzRow {
  float lse2, g, gh;
  int tgt;
};

template <typename T, bool GENERAL, bool OUT32>
__global__ __launch_bounds__(kDzThreads, 1) void dense_dz16_kernel(DzParams p) {
  using Fast = DmaLogitTile16<T, kDz16WV, kDz16WT, kDzNWV, kDzNWT>;
  extern __shared__ __align__(16) unsigned char smem[];
  float* s_addend = reinterpret_cast<float*>(smem + Fast::LDS_BYTES);                                   // [2][256]
  DzRow* s_rows = reinterpret_cast<DzRow*>(smem + Fast::LDS_BYTES + 2 * kDzTile * 4);                    // [256]
  unsigned char* s_stage = smem + Fast::LDS_BYTES + 2 * kDzTile * 4 + kDzTile * sizeof(DzRow);           // [8 waves]

  const int xcd = blockIdx.x & 7;
  const int slot = blockIdx.x >> 3;
  if (slot >= p.items_per_xcd) return;
  const int item = xcd * p.items_per_xcd + slot;
  if (item >= p.nitems) return;
  const int rb = item / p.nsplit;
  const int split = item % p.nsplit;
  const int vt_begin = static_cast<int>((static_cast<int64_t>(p.nvt) * split) / p.nsplit);
  const int vt_end = static_cast<int>((static_cast<int64_t>(p.nvt) * (split + 1)) / p.nsplit);
  if (vt_begin >= vt_end) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wv = wave / kDzNWT;
  const int wt = wave % kDzNWT;
  const int r16 = lane & 15;
  const int kq = lane >> 4;
  const int64_t t0 = static_cast<int64_t>(rb) * kDzTile;

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
  auto set_class_tile = [&](int vt) {
    const int64_t v0 = static_cast<int64_t>(vt) * kDzTile;
    const int left = static_cast<int>(min(p.v - v0, static_cast<int64_t>(kDzTile)));
    Fast::set_class_tile(src, reinterpret_cast<const unsigned char*>(p.c) + v0 * p.stride_cv * 2, left, wave);
  };

  unsigned char* stage = s_stage + wave * kDz16StageBytes;
  int buf = 0;
  set_class_tile(vt_begin);
  Fast::prefetch(src, smem);
  // What the rows of this workgroup need, fixed for the whole item (published by the first barrier of the main loop;
  // fetched behind the first stages of the ring, so that the two latencies overlap).
  if (tid < kDzTile) {
    const int64_t i = t0 + tid;
    DzRow r = {INFINITY, 0.0f, 0.0f, -1};
    if (i < p.b) {
      const int64_t row = p.valids ? static_cast<int64_t>(p.valids[i]) : i;
      r.lse2 = p.lse[i] * kLog2e;
      const int64_t tpos = row + p.shift;
      if (tpos < p.n_rows) {
        const int64_t t = p.targets[tpos] - p.target_offset;
        if (t >= 0 && t < p.v) r.tgt = static_cast<int>(t);
        r.g = p.grad_scale * (p.d_out_is_scalar ? p.d_out[0] : p.d_out[tpos]);
        r.gh = r.g + ((p.d_lse != nullptr) ? p.d_lse[tpos] : 0.0f);
      }
    }
    s_rows[tid] = r;
  }

  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int64_t v0 = static_cast<int64_t>(vt) * kDzTile;
    float* addend = s_addend + (vt & 1) * kDzTile;
    if (GENERAL) {
      if (tid < kDzTile) {  // published by the barriers of the main loop
        const int64_t vg = v0 + tid;
        float a = -INFINITY;
        if (vg < p.v) a = (p.bias != nullptr) ? Elem<T>::to_float(p.bias[vg]) : 0.0f;
        addend[tid] = a;
      }
    }
    f32x4 acc[kDz16WV][kDz16WT];
    Fast::run(acc, src, smem, static_cast<int>(p.d), buf, vt == vt_begin, [&] {
      if (vt + 1 < vt_end) set_class_tile(vt + 1);
    });

    const int cls0 = static_cast<int>(v0) + wv * (16 * kDz16WV);  // first class of this wave
    const float* wave_addend = addend + wv * (16 * kDz16WV);
    const int sw = (r16 >> 1) & 7;  // 16-byte chunks of a staged row are XOR-swizzled with (row >> 1) & 7
    // (left to itself the compiler forms the row part of every store address before the tile loop, holds the pairs
    // of registers through the main loop by spilling them, and the reload at the top of the epilogue waits for
    // the loads just issued for the next tile)
    int64_t wrow0 = t0 + wt * (16 * kDz16WT);  // first row of this wave
    asm volatile("" : "+s"(wrow0));
    constexpr int kEs = OUT32 ? 4 : 2;                  // bytes per stored element
    constexpr int kViPer = kDzStageRow / (16 * kEs);    // 16-class blocks per staged row (4, or 2 for fp32)
    constexpr int kParts = kDz16WV / kViPer;            // staged blocks per row block
    constexpr int kPieceElems = 16 / kEs;               // elements per 16-byte piece
#pragma unroll
    for (int ti = 0; ti < kDz16WT; ++ti) {
      const DzRow rr = s_rows[wt * (16 * kDz16WT) + ti * 16 + r16];
#pragma unroll
      for (int vh = 0; vh < kParts; ++vh) {
        // The gradients of one staged block.  One copy of the arithmetic per answer to "soft-capped?".
        auto stage_block = [&](auto capped) {
#pragma unroll
          for (int vj = 0; vj < kViPer; ++vj) {
            const int vi = vh * kViPer + vj;
            float dzv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int cl = vi * 16 + 4 * kq + r;
              float x = acc[vi][ti][r];
              bool dead = false;
              if (GENERAL) {
                const float add = wave_addend[cl];
                dead = (add == -INFINITY);
                x = dead ? 0.0f : x + add;
              }
              float s2, damp = 1.0f;
              if (decltype(capped)::value) {
                const float t = __builtin_amdgcn_exp2f(x * p.sc.in_scale);
                const float w = __builtin_amdgcn_rcpf(1.0f + t);
                const float th = 1.0f - 2.0f * w;
                s2 = p.sc.out_scale * th;
                damp = 1.0f - th * th;
              } else {
                s2 = x * kLog2e;
              }
              const float pr = __builtin_amdgcn_exp2f(s2 - rr.lse2);
              float dz = pr * rr.gh - ((cls0 + cl == rr.tgt) ? rr.g : 0.0f);
              if (decltype(capped)::value) dz *= damp;
              dzv[r] = dead ? 0.0f : dz;
            }
            const int col = (vj * 16 + 4 * kq) * kEs;  // byte inside the staged row
            unsigned char* dst = stage + r16 * kDzStageRow + ((((col >> 4) ^ sw) << 4) | (col & 15));
            if (OUT32) {
              *reinterpret_cast<float4*>(dst) = make_float4(dzv[0], dzv[1], dzv[2], dzv[3]);
            } else {
              uint2 pk;
              pk.x = Elem<T>::pack2(dzv[0], dzv[1]);
              pk.y = Elem<T>::pack2(dzv[2], dzv[3]);
              *reinterpret_cast<uint2*>(dst) = pk;
            }
          }
        };
        if (p.sc.on) {
          stage_block(std::true_type{});
        } else {
          stage_block(std::false_type{});
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the block is private to this wave: no barrier
        // 16 rows x 128 bytes leave as 16-byte pieces: one instruction covers 8 rows of 128 contiguous bytes
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const int j = lane + 64 * k;
          const int row = j >> 3;
          const int pc = j & 7;
          const uint4 val = *reinterpret_cast<const uint4*>(stage + row * kDzStageRow + ((pc ^ ((row >> 1) & 7)) << 4));
          const int64_t gi = wrow0 + ti * 16 + row;
          const int64_t gcol = static_cast<int64_t>(cls0) + vh * (16 * kViPer) + pc * kPieceElems;
          if (gi < p.b) {
            unsigned char* dst = static_cast<unsigned char*>(p.dz) + (gi * p.ldz + gcol) * kEs;
            if (!GENERAL || gcol + kPieceElems <= p.v || (p.pad_store && gcol + kPieceElems <= p.ldz)) {
              *reinterpret_cast<uint4*>(dst) = val;
            } else if (OUT32) {
              const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (gcol + i < p.v) reinterpret_cast<uint32_t*>(dst)[i] = w[i];
            } else {
              const uint32_t w[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
              for (int i = 0; i < 8; ++i)
                if (gcol + i < p.v) reinterpret_cast<uint16_t*>(dst)[i] = static_cast<uint16_t>(w[i >> 1] >> ((i & 1) * 16));
            }
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // reads done before the next block is staged
      }
    }
  }
  // the loads issued under the last tile (its own first stages once more) must land before the workgroup ends
  wait_vmcnt<0>();
}

int dense_dz_launch(const void* e, const void* c, const void* bias,
                    const float* lse, const float* d_out, int d_out_is_scalar, const float* d_lse,
                    const int32_t* valids, const int64_t* targets,
                    void* dz, int64_t ldz, int dz_is_fp32, int pad_store,
                    int64_t n_rows, int64_t b, int64_t v, int64_t d,
                    int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                    float grad_scale, int64_t shift, int64_t target_offset,
                    float softcap, int dtype, hipStream_t stream) {
  if (b < 0 || v <= 0 || d <= 0 || n_rows < 0 || shift < 0 || ldz < v) return CCE_ERR_INVALID_ARGUMENT;
  if (b == 0) return CCE_OK;
  if (e == nullptr || c == nullptr || lse == nullptr || d_out == nullptr || targets == nullptr || dz == nullptr)
    return CCE_ERR_INVALID_ARGUMENT;
  if (valids == nullptr && b > n_rows) return CCE_ERR_INVALID_ARGUMENT;
  if (d > (1 << 30) || v > (int64_t(1) << 31) - 512) return CCE_ERR_INVALID_ARGUMENT;
  if (dtype != CCE_DTYPE_BF16 && dtype != CCE_DTYPE_F16) return CCE_ERR_UNSUPPORTED_DTYPE;
  // direct-to-LDS main loop and 16-byte stores only
  if (!aligned16(e) || !aligned16(c) || !aligned16(dz) || d % kDmaBK != 0 || stride_e % 8 != 0 ||
      stride_cv % 8 != 0 || stride_cd != 1 || ldz % (dz_is_fp32 ? 4 : 8) != 0)
    return CCE_ERR_MISALIGNED;

  DzParams p;
  p.e = static_cast<const uint16_t*>(e);
  p.c = static_cast<const uint16_t*>(c);
  p.bias = static_cast<const uint16_t*>(bias);
  p.valids = valids;
  p.lse = lse;
  p.d_out = d_out;
  p.d_lse = d_lse;
  p.targets = targets;
  p.dz = dz;
  p.ldz = ldz;
  p.n_rows = n_rows;
  p.b = b;
  p.v = v;
  p.d = d;
  p.stride_e = stride_e;
  p.stride_cv = stride_cv;
  p.shift = shift;
  p.target_offset = target_offset;
  p.grad_scale = grad_scale;
  p.d_out_is_scalar = d_out_is_scalar;
  p.pad_store = pad_store;
  p.nrb = static_cast<int>((b + kDzTile - 1) / kDzTile);
  p.nvt = static_cast<int>((v + kDzTile - 1) / kDzTile);
  p.nsplit = choose_span_count(p.nrb, p.nvt);
  p.nitems = p.nrb * p.nsplit;
  p.items_per_xcd = (p.nitems + 7) / 8;
  p.sc = make_softcap(softcap);

  using FastB = DmaLogitTile<BF16, kDzWV, kDzWT, kDzNWV, kDzNWT>;
  const int lds = FastB::LDS_BYTES + 2 * kDzTile * 4;
  const int lds16 = lds + kDzTile * static_cast<int>(sizeof(DzRow)) + kDzNWV * kDzNWT * kDz16StageBytes;
  const bool general = (bias != nullptr) || (v % kDzTile != 0);
  // the 16 x 16 x 32 kernel addresses rows by 32-bit byte offsets and streams at least two stages per tile
  const bool k16 = (d >= 2 * kDmaBK) && (n_rows * stride_e * 2 < (int64_t(1) << 32)) &&
                   (256 * stride_cv * 2 < (int64_t(1) << 32));
  const int grid = p.items_per_xcd * 8;
  hipError_t err;
#define CCE_LAUNCH_DZ2(TT, GE, O32)                                                               \
  do {                                                                                            \
    if (k16) {                                                                                    \
      auto kern = dense_dz16_kernel<TT, GE, O32>;                                                 \
      static LdsLimitOnce lds_limit;                                                              \
      err = lds_limit.set(kern, lds16);                                                           \
      if (err != hipSuccess) return status_from_hip(err);                                         \
      hipLaunchKernelGGL(kern, dim3(grid), dim3(kDzThreads), lds16, stream, p);                   \
    } else {                                                                                      \
      auto kern = dense_dz_kernel<TT, GE, O32>;                                                   \
      static LdsLimitOnce lds_limit;                                                              \
      err = lds_limit.set(kern, lds);                                                             \
      if (err != hipSuccess) return status_from_hip(err);                                         \
      hipLaunchKernelGGL(kern, dim3(grid), dim3(kDzThreads), lds, stream, p);                     \
    }                                                                                             \
  } while (0)
#define CCE_LAUNCH_DZ(TT, GE)                                                                     \
  do {                                                                                            \
    if (dz_is_fp32) CCE_LAUNCH_DZ2(TT, GE, true); else CCE_LAUNCH_DZ2(TT, GE, false);             \
  } while (0)
  if (dtype == CCE_DTYPE_BF16) {
    if (general) CCE_LAUNCH_DZ(BF16, true); else CCE_LAUNCH_DZ(BF16, false);
  } else {
    if (general) CCE_LAUNCH_DZ(F16, true); else CCE_LAUNCH_DZ(F16, false);
  }
#undef CCE_LAUNCH_DZ
#undef CCE_LAUNCH_DZ2
  return status_from_hip(hipGetLastError());
}

}  // namespace cce

extern "C" int cce_backward_dz(const void* e, const void* c, const void* bias,
                               const float* lse, const float* d_out, int d_out_is_scalar, const float* d_lse,
                               const int32_t* valids, const int64_t* targets,
                               void* dz, int64_t ldz, int dz_is_fp32,
                               int64_t n_rows, int64_t b, int64_t v, int64_t d,
                               int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                               float grad_scale, int64_t shift, int64_t target_offset,
                               float softcap, int dtype, void* stream) {
  return cce::dense_dz_launch(e, c, bias, lse, d_out, d_out_is_scalar, d_lse, valids, targets, dz, ldz, dz_is_fp32, 0,
                              n_rows, b, v, d, stride_e, stride_cv, stride_cd, grad_scale, shift, target_offset, softcap,
                              dtype, static_cast<hipStream_t>(stream));
}
