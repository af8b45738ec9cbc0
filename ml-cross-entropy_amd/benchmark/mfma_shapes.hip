// mfma_shapes: what the matrix pipes of one gfx950 chip sustain from registers alone -- no LDS, no memory -- for the
// two dense 16-bit MFMA shapes, several issue orders of the same 128 x 64 wave tile (the forward kernel's), and
// operands of full entropy against operands of zeros.  The chip runs these loops against its power limit, not
// against its issue rate: the figure with zeros is the issue-bound one, the figures with random operands are what
// the power limit leaves, and they differ by instruction shape.  This is the measurement behind the choice of
// 16 x 16 x 32 MFMAs in csrc/cce_common.h (DmaLogitTile16).
//
// build:  make -C ml-cross-entropy_amd/csrc probes     (-> ml-cross-entropy_amd/benchmark/mfma_shapes)
// run:    ml-cross-entropy_amd/benchmark/mfma_shapes [iterations, default 20000]
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t hash(uint32_t s) {
  s ^= s >> 16; s *= 0x7feb352du; s ^= s >> 15; s *= 0x846ca68bu; s ^= s >> 16; return s;
}
// random bf16 with |x| ~ scale (sign, 7 random mantissa bits, small exponent spread); scale 0 -> zeros
__device__ __forceinline__ bf16x8 rnd8(uint32_t seed, float scale) {
  bf16x8 v;
  for (int i = 0; i < 8; ++i) {
    uint32_t h = hash(seed * 8u + i);
    float f = ((h & 0xffff) + (h >> 16)) / 65536.0f - 1.0f;  // triangular in (-1, 1)
    v[i] = (__bf16)(f * scale);
  }
  return v;
}

constexpr int NSET = 4;
// MODE 0: 32x32x16, 4x2 blocks, vi outer (shipped order); 1: snake; 2: ti outer; 3: 16x16x32, 8x4 blocks
template <int MODE>
__global__ __launch_bounds__(512, 1) void k(float* out, int iters, float sa, float sb) {
  const uint32_t t = blockIdx.x * 512 + threadIdx.x;
  if (MODE < 3) {
    bf16x8 a[NSET][4], b[NSET][2];
    for (int s = 0; s < NSET; ++s) {
      for (int i = 0; i < 4; ++i) a[s][i] = rnd8(t * 64 + s * 8 + i, sa);
      for (int i = 0; i < 2; ++i) b[s][i] = rnd8(t * 64 + s * 8 + 4 + i, sb);
    }
    f32x16 acc[4][2];
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 2; ++j) for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int s = 0; s < NSET; ++s) {
        if (MODE == 0) {
#pragma unroll
          for (int vi = 0; vi < 4; ++vi)
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
              acc[vi][ti] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s][vi], b[s][ti], acc[vi][ti], 0, 0, 0);
        } else if (MODE == 1) {
#pragma unroll
          for (int vi = 0; vi < 4; ++vi)
#pragma unroll
            for (int tj = 0; tj < 2; ++tj) {
              const int ti = (vi & 1) ? 1 - tj : tj;
              acc[vi][ti] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s][vi], b[s][ti], acc[vi][ti], 0, 0, 0);
            }
        } else {
#pragma unroll
          for (int ti = 0; ti < 2; ++ti)
#pragma unroll
            for (int vi = 0; vi < 4; ++vi)
              acc[vi][ti] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s][vi], b[s][ti], acc[vi][ti], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    float sum = 0;
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 2; ++j) for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
    out[t] = sum;
  } else {
    // the same 128 x 64 wave tile from 16x16x32 instructions: 8 x 4 blocks of 4 registers; one "set" = 32 columns
    constexpr int NS2 = 2;
    bf16x8 a[NS2][8], b[NS2][4];
    for (int s = 0; s < NS2; ++s) {
      for (int i = 0; i < 8; ++i) a[s][i] = rnd8(t * 64 + s * 16 + i, sa);
      for (int i = 0; i < 4; ++i) b[s][i] = rnd8(t * 64 + s * 16 + 8 + i, sb);
    }
    f32x4 acc[8][4];
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 4; ++j) for (int r = 0; r < 4; ++r) acc[i][j][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int rep = 0; rep < NSET / NS2; ++rep)
#pragma unroll
      for (int s = 0; s < NS2; ++s) {
        if (MODE == 3) {
#pragma unroll
        for (int vi = 0; vi < 8; ++vi)
#pragma unroll
          for (int ti = 0; ti < 4; ++ti)
            acc[vi][ti] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][vi], b[s][ti], acc[vi][ti], 0, 0, 0);
        } else if (MODE == 4) {
#pragma unroll
        for (int ti = 0; ti < 4; ++ti)
#pragma unroll
          for (int vi = 0; vi < 8; ++vi)
            acc[vi][ti] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][vi], b[s][ti], acc[vi][ti], 0, 0, 0);
        } else {
#pragma unroll
        for (int vi = 0; vi < 8; ++vi)
#pragma unroll
          for (int tj = 0; tj < 4; ++tj) {
            const int ti = (vi & 1) ? 3 - tj : tj;
            acc[vi][ti] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][vi], b[s][ti], acc[vi][ti], 0, 0, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    float sum = 0;
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 4; ++j) for (int r = 0; r < 4; ++r) sum += acc[i][j][r];
    out[t] = sum;
  }
}

template <int MODE>
static void run(const char* name, int threads, float sa, float sb, float* out, int iters) {
  hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
  float best = 1e9, sum = 0; const int reps = 4;
  for (int r = 0; r < reps + 1; ++r) {
    hipEventRecord(e0);
    hipLaunchKernelGGL(k<MODE>, dim3(256), dim3(threads), 0, 0, out, iters, sa, sb);
    hipEventRecord(e1); hipEventSynchronize(e1);
    float ms; hipEventElapsedTime(&ms, e0, e1);
    if (r) { sum += ms; if (ms < best) best = ms; }
  }
  // flops per wave and iteration: NSET sets; MODE<3: 8 MFMAs of 32768 each = 262144 per 16-col set; MODE 3: one set = 32 MFMAs x 16384 = 524288 (32 cols)
  const double per_set = (MODE < 3) ? 8 * 32768.0 : 32 * 16384.0;
  const double fl = 256.0 * (threads / 64) * iters * NSET * per_set;
  printf("%-34s waves/SIMD %d  a %.3g b %.3g : avg %.3f ms  %.1f TFLOP/s (%.1f%%)\n", name, threads / 256, sa, sb, sum / reps,
         fl / (sum / reps) / 1e9, fl / (sum / reps) / 1e9 / 25.166);
  fflush(stdout);
}

int main(int argc, char** argv) {
  int iters = argc > 1 ? atoi(argv[1]) : 20000;
  float* out;
  if (hipMalloc(&out, 256 * 512 * 4) != hipSuccess) { printf("no device memory\n"); return 1; }
  run<0>("32x32x16 vi-outer", 512, 1.0f, 0.02f, out, iters);
  run<1>("32x32x16 snake", 512, 1.0f, 0.02f, out, iters);
  run<2>("32x32x16 ti-outer", 512, 1.0f, 0.02f, out, iters);
  run<3>("16x16x32 8x4 vi-outer", 512, 1.0f, 0.02f, out, iters / 2);
  run<4>("16x16x32 8x4 ti-outer", 512, 1.0f, 0.02f, out, iters / 2);
  run<5>("16x16x32 8x4 snake", 512, 1.0f, 0.02f, out, iters / 2);
  run<3>("16x16x32 8x4 vi-outer zeros", 512, 0.0f, 0.0f, out, iters / 2);
  run<0>("32x32x16 vi-outer zeros", 512, 0.0f, 0.0f, out, iters);
  run<0>("32x32x16 vi-outer a=0", 512, 0.0f, 0.02f, out, iters);
  run<0>("32x32x16 vi-outer b=0", 512, 1.0f, 0.0f, out, iters);
  run<0>("32x32x16 vi-outer 1 wave/SIMD", 256, 1.0f, 0.02f, out, iters);
  run<0>("32x32x16 vi-outer (again)", 512, 1.0f, 0.02f, out, iters);
  return 0;
}
