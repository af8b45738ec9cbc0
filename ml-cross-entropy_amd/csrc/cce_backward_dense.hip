// cce_backward_dense: the unfiltered backward (gradient filter off) in one call.
//
// With every entry of dz = d loss / d logits in play the two gradient products are dense:
//     dE[rows] = dz . C          dC = dz^T . E[rows]          dBias = column sums of dz
// The reference forms them inside its one kernel with atomics on dE and dC
// (cut_cross_entropy/cce_backward.py:258-310).  On this chip a tile of dz can feed register-resident
// accumulators of only one of the two outputs at a time (a 256-row slab of dE or dC over D = 2304 .. 4096
// columns is 2.4 .. 4 MB of fp32, against 0.5 MB of registers per compute unit) and global float atomics are
// an order of magnitude too slow, so the vocabulary is walked in chunks and per chunk
//   1. dense_dz_kernel    recomputes the logits of the chunk and writes dz [B, vc] in the input type
//                         (the chunk is sized to stay in the last-level cache),
//   2. dense_dc_kernel    dC[chunk] = dz^T . E : complete for these classes, written once,
//      (2 and 3 are tiles of one launch, dense_products_kernel)
//   3. dense_de_kernel    dE += dz . C[chunk]  : accumulated across the chunks in d_e itself, in fp32 when the caller
//                         asked for an fp32 dE, else as d_e (16 bit) plus a 16-bit compensation term in the workspace,
//   4. dz_colsum_kernel   dBias[chunk], when wanted.
// Where the rows are many against the classes (a vocabulary shard: 65536 rows x 19008 classes) the walk goes over
// blocks of ROWS instead, each with the whole vocabulary: dE of a block is then complete after its one launch (written
// once, no compensation buffer of [b, d]) and it is dC that is carried from block to block, as a pair of 16-bit
// numbers with a [v, d] compensation buffer.  Same kernels, the roles of the two outputs exchanged.
// Both products run on the tile loop of cce_tile4.h (direct-to-LDS loads, LDS transpose reads for the
// operand whose reduction index is the row index).  Everything is enqueued on the caller's stream; nothing
// is allocated, no host synchronisation.
#include <queue>
#include <vector>

#include "cce_dense.h"
#include "cce_tile4.h"

namespace cce {

struct ProductParams {
  const uint16_t* dz;   // [b][ldz]
  int64_t ldz;
  const uint16_t* c;    // first class of the chunk
  int64_t stride_cv;
  const uint16_t* e;
  int64_t stride_e;
  const int32_t* valids;
  float* de_f32;        // dE accumulated in fp32, in the caller's float d_e (rows of e, through valids); or nullptr:
  uint16_t* de_hi;      // dE accumulated as a pair of 16-bit values hi + lo: hi is the caller's d_e in the input type
  uint16_t* de_lo;      //   (rows of e), lo the compensation term in the workspace ([b][d], rows by valid-row number)
  int64_t ld_de;        // row stride of d_e (elements)
  int first_chunk;      // nothing accumulated yet: the pair is written, not read (de_lo == nullptr: the 16-bit d_e is
                        //   complete with this launch and written alone)
  void* d_c;            // first class of the chunk
  int64_t ld_dc;        // row stride of d_c (elements)
  int dc_fp32;
  int dc_accumulate;    // d_c (fp32) is added to, not written
  uint16_t* dc_lo;      // a 16-bit d_c carried over blocks of rows as a pair hi + lo: hi is d_c, lo this [n_cls][d]
  int dc_first;         //   compensation term in the workspace (nullptr: d_c is written once); the first block writes the pair
  int de_rows_by_number;  // the fp32 d_e is indexed by valid-row number (a [b, d] accumulator), not by row of e
  int64_t b;
  int d;
  int n_cls;            // classes in the chunk
  int tiles_n;          // column tiles of either output
  int dc_tiles, dc_per_xcd;  // tiles of dC, slots per XCD
  int de_tiles, de_per_xcd;
  int de_first;              // the dE tiles have the longer reduction and take the first block ids
};

constexpr int kProdThreads = 256;  // four waves, one per SIMD

// Tile `block` of a group of `tiles` tiles (tiles_n column tiles wide).  Block ids that land on one XCD get
// consecutive places in an order that keeps the 32 tiles an XCD works on at a time on few operand panels: a tile
// streams one A panel (its row of tiles) and one B panel (its column) through the XCD's L2, so 32 tiles of one or
// two rows of a wide output need 2 + 16 panels where a block of 4 x 8 tiles needs 12.  The columns are therefore
// cut into groups of at most 8 (as equal as possible), and the order walks a group row by row before it moves to
// the next group (E [15356, 4096] x C [128256, 4096], 16 column tiles: backward 39.3 -> 38.1 ms).
__device__ __forceinline__ bool product_tile_of(int block, int tiles, int per_xcd, int tiles_n, int& tm, int& tn) {
  const int xcd = block & 7;
  const int slot = block >> 3;
  int lin = xcd * per_xcd + slot;
  if (lin >= tiles) return false;
  const int tiles_m = tiles / tiles_n;
  const int groups = (tiles_n + 7) / 8;
  const int narrow = tiles_n / groups;          // width of the narrow groups; the first `wide` groups have one more
  const int wide = tiles_n - narrow * groups;
  const int in_wide = wide * tiles_m * (narrow + 1);
  int width, first_col;
  if (lin < in_wide) {
    width = narrow + 1;
    const int grp = lin / (tiles_m * width);
    lin -= grp * tiles_m * width;
    first_col = grp * width;
  } else {
    width = narrow;
    lin -= in_wide;
    const int grp = lin / (tiles_m * width);
    lin -= grp * tiles_m * width;
    first_col = wide * (narrow + 1) + grp * width;
  }
  tm = lin / width;
  tn = first_col + (lin - tm * width);
  return true;
}

// dE[row][col] += sum_class dz[row][class] * C[class][col]
template <typename T, bool SPLIT_DE>
__device__ __forceinline__ void dense_de_tile(const ProductParams& p, int tm, int tn, unsigned char* smem) {
  using Tile = Tile4<T, false, true>;
  typename Tile::Geometry g = Tile::geometry(smem);
  const int64_t m0 = static_cast<int64_t>(tm) * Tile::TILE;
  const int n0 = tn * Tile::TILE;

  typename Tile::Source s;
#pragma unroll
  for (int q = 0; q < Tile::NQ1; ++q) {
    int64_t i = m0 + Tile::row_direct(q, g.wave, g.lane);
    i = (i < p.b) ? i : p.b - 1;  // rows past the end repeat the last one; their results are dropped
    s.a_row[q] = p.dz + i * p.ldz + Tile::chunk_direct(g.wave, g.lane);
  }
  s.b_row[0] = nullptr;
  s.a_km = nullptr;
  s.a_stride = 0;
  // (columns past d: the last chunk inside the matrix once more; what they feed is dropped below)
  s.b_km = p.c + min(n0 + Tile::chunk_kmajor(g.wave, g.lane), p.d - 8);
  s.b_stride = p.stride_cv;
  s.b_rows = nullptr;
  s.k_total = p.n_cls;

  // What memory holds of a piece so far, fetched ahead of its use.
  struct Old {
    int64_t re;   // the piece's row of e (-1: the piece lies outside the matrix)
    uint4 a, b;   // fp32 dE: the eight sums; a 16-bit dE: the hi and the lo halves of the eight sums
  };
  auto fetch = [&](int row, int col) {
    Old o;
    o.re = -1;
    o.a = make_uint4(0u, 0u, 0u, 0u);
    o.b = make_uint4(0u, 0u, 0u, 0u);
    const int64_t ri = m0 + row;          // valid-row number
    const int cg = n0 + col;
    if (ri >= p.b || cg >= p.d) return o;
    o.re = (p.valids != nullptr && !p.de_rows_by_number) ? static_cast<int64_t>(p.valids[ri]) : ri;
    if (!SPLIT_DE) {
      const uint4* src = reinterpret_cast<const uint4*>(p.de_f32 + o.re * p.ld_de + cg);
      o.a = src[0];
      o.b = src[1];
    } else if (!p.first_chunk) {  // (never with de_lo == nullptr: a d_e written alone is a first chunk)
      o.a = *reinterpret_cast<const uint4*>(p.de_hi + o.re * p.ld_de + cg);
      o.b = *reinterpret_cast<const uint4*>(p.de_lo + ri * p.d + cg);
    }
    return o;
  };
  f32x16 acc[Tile::WM][Tile::WN];
  typename Tile::Loop loop = Tile::plan(s, g);
  typename Tile::Ids ids;
  typename Tile::Ptrs ptrs;
  Tile::prefetch(s, loop, ptrs, ids, g);
  Tile::run(acc, s, loop, ptrs, ids, smem, g);

  // (fetching the first slabs before the main loop instead would hold 80 registers across it: they spill)
  typename Tile::template Rmw<Old> rmw;
  Tile::rmw_begin(rmw, g, fetch);
  Tile::for_each_row_piece_rmw(acc, smem, g, rmw, fetch, [&](int row, int col, const float (&v)[8], const Old& o) {
    if (o.re < 0) return;
    const int64_t ri = m0 + row;
    const int cg = n0 + col;
    if (!SPLIT_DE) {
      float4* dst = reinterpret_cast<float4*>(p.de_f32 + o.re * p.ld_de + cg);
      float4 a = __builtin_bit_cast(float4, o.a), b = __builtin_bit_cast(float4, o.b);
      a.x += v[0]; a.y += v[1]; a.z += v[2]; a.w += v[3];
      b.x += v[4]; b.y += v[5]; b.z += v[6]; b.w += v[7];
      dst[0] = a;
      dst[1] = b;
    } else {
      // value so far = hi + lo (two 16-bit numbers: 16 bits of mantissa, where one would round the sum of a few
      // dozen chunks eight bits short); the new hi is the rounded total, so the last chunk leaves d_e final
      uint4* hi_ptr = reinterpret_cast<uint4*>(p.de_hi + o.re * p.ld_de + cg);
      uint4* lo_ptr = reinterpret_cast<uint4*>(p.de_lo + ri * p.d + cg);
      const uint32_t hw[4] = {o.a.x, o.a.y, o.a.z, o.a.w}, lw[4] = {o.b.x, o.b.y, o.b.z, o.b.w};
      uint32_t ho[4], lo_out[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float t[2], rest[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
          t[h] = (Elem<T>::to_float(static_cast<uint16_t>(hw[k] >> (16 * h))) +
                  Elem<T>::to_float(static_cast<uint16_t>(lw[k] >> (16 * h)))) + v[2 * k + h];
        ho[k] = Elem<T>::pack2(t[0], t[1]);
#pragma unroll
        for (int h = 0; h < 2; ++h) rest[h] = t[h] - Elem<T>::to_float(static_cast<uint16_t>(ho[k] >> (16 * h)));
        lo_out[k] = Elem<T>::pack2(rest[0], rest[1]);
      }
      *hi_ptr = make_uint4(ho[0], ho[1], ho[2], ho[3]);
      if (p.de_lo != nullptr) *lo_ptr = make_uint4(lo_out[0], lo_out[1], lo_out[2], lo_out[3]);
    }
  });
}

// dC[class][col] = sum_row dz[row][class] * E[row][col]; GATHER: the rows of E come through valids
template <typename T, bool GATHER>
__device__ __forceinline__ void dense_dc_tile(const ProductParams& p, int tm, int tn, unsigned char* smem) {
  using Tile = Tile4<T, true, true, GATHER>;
  typename Tile::Geometry g = Tile::geometry(smem);
  const int m0 = tm * Tile::TILE;
  const int n0 = tn * Tile::TILE;

  typename Tile::Source s;
  s.a_row[0] = nullptr;
  s.b_row[0] = nullptr;
  const int chunk = Tile::chunk_kmajor(g.wave, g.lane);
  // (columns past the matrix: the last chunk inside it once more; what they feed is dropped below)
  s.a_km = p.dz + min(static_cast<int64_t>(m0 + chunk), p.ldz - 8);
  s.a_stride = p.ldz;
  s.b_km = p.e + min(n0 + chunk, p.d - 8);
  s.b_stride = p.stride_e;
  s.b_rows = p.valids;
  s.k_total = static_cast<int>(p.b);

  f32x16 acc[Tile::WM][Tile::WN];
  typename Tile::Loop loop = Tile::plan(s, g);
  typename Tile::Ids ids;
  typename Tile::Ptrs ptrs;
  Tile::prefetch(s, loop, ptrs, ids, g);
  Tile::run(acc, s, loop, ptrs, ids, smem, g);

  if (p.dc_lo != nullptr) {
    // a 16-bit dC carried over blocks of rows: value so far = hi + lo, as dE is carried over chunks of classes
    struct Old {
      int ok;
      uint4 a, b;
    };
    auto fetch = [&](int row, int col) {
      Old o;
      o.ok = 0;
      o.a = make_uint4(0u, 0u, 0u, 0u);
      o.b = make_uint4(0u, 0u, 0u, 0u);
      const int cls = m0 + row;
      const int cg = n0 + col;
      if (cls >= p.n_cls || cg >= p.d) return o;
      o.ok = 1;
      if (!p.dc_first) {
        o.a = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(p.d_c) + static_cast<int64_t>(cls) * p.ld_dc + cg);
        o.b = *reinterpret_cast<const uint4*>(p.dc_lo + static_cast<int64_t>(cls) * p.d + cg);
      }
      return o;
    };
    typename Tile::template Rmw<Old> rmw;
    Tile::rmw_begin(rmw, g, fetch);
    Tile::for_each_row_piece_rmw(acc, smem, g, rmw, fetch, [&](int row, int col, const float (&v)[8], const Old& o) {
      if (!o.ok) return;
      const int cls = m0 + row;
      const int cg = n0 + col;
      uint4* hi_ptr = reinterpret_cast<uint4*>(static_cast<uint16_t*>(p.d_c) + static_cast<int64_t>(cls) * p.ld_dc + cg);
      uint4* lo_ptr = reinterpret_cast<uint4*>(p.dc_lo + static_cast<int64_t>(cls) * p.d + cg);
      const uint32_t hw[4] = {o.a.x, o.a.y, o.a.z, o.a.w}, lw[4] = {o.b.x, o.b.y, o.b.z, o.b.w};
      uint32_t ho[4], lo_out[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float t[2], rest[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
          t[h] = (Elem<T>::to_float(static_cast<uint16_t>(hw[k] >> (16 * h))) +
                  Elem<T>::to_float(static_cast<uint16_t>(lw[k] >> (16 * h)))) + v[2 * k + h];
        ho[k] = Elem<T>::pack2(t[0], t[1]);
#pragma unroll
        for (int h = 0; h < 2; ++h) rest[h] = t[h] - Elem<T>::to_float(static_cast<uint16_t>(ho[k] >> (16 * h)));
        lo_out[k] = Elem<T>::pack2(rest[0], rest[1]);
      }
      *hi_ptr = make_uint4(ho[0], ho[1], ho[2], ho[3]);
      *lo_ptr = make_uint4(lo_out[0], lo_out[1], lo_out[2], lo_out[3]);
    });
    return;
  }
  Tile::for_each_row_piece(acc, smem, g, [&](int row, int col, const float (&v)[8]) {
    const int cls = m0 + row;
    const int cg = n0 + col;
    if (cls >= p.n_cls || cg >= p.d) return;
    const int64_t off = static_cast<int64_t>(cls) * p.ld_dc + cg;
    if (p.dc_fp32) {
      float4* dst = reinterpret_cast<float4*>(static_cast<float*>(p.d_c) + off);
      float4 a = make_float4(v[0], v[1], v[2], v[3]), b = make_float4(v[4], v[5], v[6], v[7]);
      if (p.dc_accumulate) {
        const float4 a0 = dst[0], b0 = dst[1];
        a.x += a0.x; a.y += a0.y; a.z += a0.z; a.w += a0.w;
        b.x += b0.x; b.y += b0.y; b.z += b0.z; b.w += b0.w;
      }
      dst[0] = a;
      dst[1] = b;
    } else {
      *reinterpret_cast<uint4*>(static_cast<uint16_t*>(p.d_c) + off) =
          make_uint4(Elem<T>::pack2(v[0], v[1]), Elem<T>::pack2(v[2], v[3]), Elem<T>::pack2(v[4], v[5]), Elem<T>::pack2(v[6], v[7]));
    }
  });
}

// Both products of one chunk in one launch.  Blocks are handed to compute units in id order as units fall free:
// the kind of tile with the longer reduction (dC: all B rows; dE: the classes of the chunk) takes the first block
// ids, so that the shorter tiles fill the last round of the longer ones.
template <typename T, bool SPLIT_DE>
__global__ __launch_bounds__(kProdThreads, 1) void dense_products_kernel(ProductParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int first_blocks = (p.de_first ? p.de_per_xcd : p.dc_per_xcd) * 8;
  const bool first = static_cast<int>(blockIdx.x) < first_blocks;
  const int block = first ? blockIdx.x : blockIdx.x - first_blocks;
  int tm, tn;
  if (first != (p.de_first != 0)) {
    if (!product_tile_of(block, p.dc_tiles, p.dc_per_xcd, p.tiles_n, tm, tn)) return;
    if (p.valids != nullptr) {
      dense_dc_tile<T, true>(p, tm, tn, smem);
    } else {
      dense_dc_tile<T, false>(p, tm, tn, smem);
    }
  } else {
    if (!product_tile_of(block, p.de_tiles, p.de_per_xcd, p.tiles_n, tm, tn)) return;
    dense_de_tile<T, SPLIT_DE>(p, tm, tn, smem);
  }
}

// dBias[class] = sum_row dz[row][class] over the chunk: 1024 threads = 16 row lanes x 64 classes.
template <typename T>
__global__ __launch_bounds__(1024) void dz_colsum_kernel(const uint16_t* dz, int64_t ldz, int64_t b, int n_cls, float* d_bias) {
  __shared__ float part[16][64];
  const int cl = threadIdx.x & 63;
  const int rl = threadIdx.x >> 6;
  const int cls = blockIdx.x * 64 + cl;
  float sum = 0.0f;
  if (cls < n_cls) {
    for (int64_t i = rl; i < b; i += 16) sum += Elem<T>::to_float(dz[i * ldz + cls]);
  }
  part[rl][cl] = sum;
  __syncthreads();
  if (rl == 0 && cls < n_cls) {
    float t = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; ++j) t += part[j][cl];  // fixed order: deterministic
    d_bias[cls] += t;
  }
}

static int64_t dense_chunk_classes_uncached(int64_t b, int64_t v, int64_t d, int64_t max_dz_bytes, bool want_de,
                                            bool want_dc);

// Rounds the product launch of one chunk takes, in units of 256 reduction steps: n_long tiles of length
// len_long and n_short tiles of len_short handed out in that order to 256 compute units as they fall free.
static double product_makespan(int64_t n_long, int64_t len_long, int64_t n_short, int64_t len_short) {
  const int cus = compute_units();
  if (len_long < len_short) {
    const int64_t n = n_long, l = len_long;
    n_long = n_short; len_long = len_short; n_short = n; len_short = l;
  }
  // greedy list scheduling over a min-heap of the units' finishing times
  std::priority_queue<int64_t, std::vector<int64_t>, std::greater<int64_t>> free_at;
  for (int i = 0; i < cus; ++i) free_at.push(0);
  int64_t worst = 0;
  auto give = [&](int64_t n, int64_t len) {
    for (int64_t t = 0; t < n; ++t) {
      const int64_t end = free_at.top() + len;
      free_at.pop();
      free_at.push(end);
      worst = end > worst ? end : worst;
    }
  };
  give(n_long, len_long);
  give(n_short, len_short);
  return static_cast<double>(worst);
}

// Classes per chunk for a dz buffer of at most `max_dz_bytes`: a multiple of 256 up to 16384 that the buffer can
// hold, chosen for the least estimated time of the whole vocabulary (whole chunks and the shorter last one): per
// chunk the dz kernel and the product launch (dC tiles with a reduction over b rows, dE tiles with a reduction
// over vc classes, the longer kind first, filling 256 compute units as they fall free).  0: the buffer cannot
// hold 256 classes.
static int64_t dense_chunk_classes(int64_t b, int64_t v, int64_t d, int64_t max_dz_bytes, bool want_de, bool want_dc) {
  // The same questions come with every step of a training loop -- the size query with the caller's dz budget, then
  // the call itself with the bytes that query answered -- so the last few answers of this thread are kept (the
  // search simulates two schedules for each of up to 64 chunk sizes: 1-3 ms of host time per question).
  struct Memo {
    int64_t b, v, d, bytes, answer;
    bool de, dc;
  };
  constexpr int kMemos = 8;
  static thread_local Memo memo[kMemos] = {};
  static thread_local int next_slot = 0;
  for (int i = 0; i < kMemos; ++i) {
    const Memo& m = memo[i];
    if (m.b == b && m.v == v && m.d == d && m.bytes == max_dz_bytes && m.de == want_de && m.dc == want_dc && m.b != 0)
      return m.answer;
  }
  const int64_t answer = dense_chunk_classes_uncached(b, v, d, max_dz_bytes, want_de, want_dc);
  memo[next_slot] = {b, v, d, max_dz_bytes, answer, want_de, want_dc};
  next_slot = (next_slot + 1) % kMemos;
  return answer;
}

// Estimated time of one chunk of vc classes in units of 256 reduction steps of a tile: the dz kernel (row_tiles x
// vc / 256 logit tiles of d / 256 units each, in rounds of 256) and the product launch.
static double chunk_cost(int64_t b, int64_t d, int64_t vc, bool want_de, bool want_dc) {
  const int64_t col_tiles = (d + 255) / 256;
  const int64_t row_tiles = (b + 255) / 256;
  const double products = product_makespan(want_dc ? vc / 256 * col_tiles : 0, row_tiles,
                                           want_de ? row_tiles * col_tiles : 0, vc / 256);
  const int64_t dz_tiles = row_tiles * (vc / 256);
  const int64_t cus = compute_units();
  const double dz = static_cast<double>((dz_tiles + cus - 1) / cus) * static_cast<double>(col_tiles);
  return products + dz + 0.25;  // the constant only breaks ties towards fewer chunks: launches queue back to back
}

static int64_t dense_chunk_classes_uncached(int64_t b, int64_t v, int64_t d, int64_t max_dz_bytes, bool want_de,
                                            bool want_dc) {
  const int64_t v_pad = (v + 255) / 256 * 256;
  int64_t top = max_dz_bytes / (b * 2) / 256 * 256;
  if (top > 16384) top = 16384;
  if (top < 256) return 0;
  if (top >= v_pad) return v_pad;
  int64_t best = top;
  double best_cost = 1e300;
  for (int64_t vc = top; vc >= 256; vc -= 256) {
    // whole chunks, then the shorter last one
    const int64_t full = v / vc;
    const int64_t rest = (v - full * vc + 255) / 256 * 256;
    double cost = static_cast<double>(full) * chunk_cost(b, d, vc, want_de, want_dc);
    if (rest > 0) cost += chunk_cost(b, d, rest, want_de, want_dc);
    if (cost < best_cost * (1.0 - 1e-9)) {
      best = vc;
      best_cost = cost;
    }
  }
  return best;
}

static int64_t align256(int64_t x) { return (x + 255) / 256 * 256; }

// How cce_backward_dense walks the [b, v] plane for a dz buffer of at most `max_dz_bytes`.
//   by classes  chunks of `unit` classes, all b rows each: dC of a chunk is complete, dE is carried over the chunks
//               (a 16-bit dE as a pair: fixed part of the workspace = its [b, d] compensation term);
//   by rows     blocks of `unit` rows, all v classes each: dE of a block is complete, dC is carried over the blocks
//               (fixed part = a [v, d] compensation term).
// Both walks take the same number of launches for the same buffer; what is carried is read and written once per
// launch, and its compensation term sits in the workspace for the whole call, so the walk goes by rows where the
// rows outnumber the classes two to one (measured, E [65536, 3584] x C [19008, 3584]: 36.1 ms and 581 MB by classes
// with 1024-class chunks, against the same 130 MB of dz by rows).  Only with 16-bit gradients: an fp32 dE is its own
// accumulator.  unit == 0: not even the smallest plan (256 classes / rows) fits.
struct DensePlan {
  bool by_rows;
  int64_t unit;
  int64_t fixed_bytes;
  int64_t dz_bytes;
};
static bool dense_walks_by_rows(int64_t b, int64_t v, bool gradients_16bit) {
  return gradients_16bit && b >= 2 * ((v + 255) / 256 * 256);
}
static DensePlan dense_plan(int64_t b, int64_t v, int64_t d, bool gradients_16bit, int64_t max_dz_bytes) {
  DensePlan pl;
  pl.by_rows = dense_walks_by_rows(b, v, gradients_16bit);
  if (pl.by_rows) {
    const int64_t v_pad = (v + 255) / 256 * 256;
    const int64_t b_pad = (b + 255) / 256 * 256;
    pl.fixed_bytes = align256(v * d * 2);
    int64_t rb = max_dz_bytes / (v_pad * 2) / 256 * 256;
    if (rb > b_pad) rb = b_pad;
    if (rb >= 256) {  // blocks of equal size: the last one is not a sliver
      const int64_t blocks = (b + rb - 1) / rb;
      rb = ((b + blocks - 1) / blocks + 255) / 256 * 256;
    }
    pl.unit = rb >= 256 ? rb : 0;
    pl.dz_bytes = align256(pl.unit * v_pad * 2);
  } else {
    pl.fixed_bytes = gradients_16bit ? align256(b * d * 2) : 0;
    pl.unit = dense_chunk_classes(b, v, d, max_dz_bytes, true, true);
    pl.dz_bytes = align256(b * pl.unit * 2);
  }
  return pl;
}

}  // namespace cce

using namespace cce;

extern "C" int64_t cce_backward_dense_workspace_bytes(int64_t b, int64_t v, int64_t d, int d_e_in_workspace,
                                                      int64_t max_dz_bytes) {
  if (b <= 0 || v <= 0 || d <= 0) return 0;
  DensePlan pl = dense_plan(b, v, d, d_e_in_workspace != 0, max_dz_bytes);
  if (pl.unit == 0) {  // the smallest plan
    const int64_t v_pad = (v + 255) / 256 * 256;
    pl.dz_bytes = align256(256 * (pl.by_rows ? v_pad : b) * 2);
  }
  return pl.fixed_bytes + pl.dz_bytes;
}

extern "C" int64_t cce_backward_dense_fixed_bytes(int64_t b, int64_t v, int64_t d, int d_e_in_workspace) {
  if (b <= 0 || v <= 0 || d <= 0) return 0;
  return dense_plan(b, v, d, d_e_in_workspace != 0, 0).fixed_bytes;
}

extern "C" int64_t cce_backward_dense_dz_bytes(int64_t b, int64_t v, int64_t d, int d_e_in_workspace, int64_t units) {
  if (b <= 0 || v <= 0 || d <= 0 || units <= 0) return 0;
  const int64_t v_pad = (v + 255) / 256 * 256;
  const int64_t b_pad = (b + 255) / 256 * 256;
  const int64_t u = (units + 255) / 256 * 256;
  if (dense_walks_by_rows(b, v, d_e_in_workspace != 0)) return (u < b_pad ? u : b_pad) * v_pad * 2;
  return b * (u < v_pad ? u : v_pad) * 2;
}

extern "C" int cce_backward_dense(const void* e, const void* c, const void* bias,
                                  const float* lse, const float* d_out, int d_out_is_scalar, const float* d_lse,
                                  const int32_t* valids, const int64_t* targets,
                                  void* d_e, void* d_c, float* d_bias,
                                  void* workspace, int64_t workspace_bytes,
                                  int64_t n_rows, int64_t b, int64_t v, int64_t d,
                                  int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                                  float grad_scale, int d_e_is_fp32, int d_c_is_fp32,
                                  int64_t shift, int64_t target_offset,
                                  float softcap, int dtype, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (b < 0 || v <= 0 || d <= 0 || n_rows < 0 || shift < 0) return CCE_ERR_INVALID_ARGUMENT;
  if (b == 0) return CCE_OK;
  if (e == nullptr || c == nullptr || lse == nullptr || d_out == nullptr || targets == nullptr)
    return CCE_ERR_INVALID_ARGUMENT;
  if (valids == nullptr && b > n_rows) return CCE_ERR_INVALID_ARGUMENT;
  if (n_rows >= (int64_t(1) << 31) || b >= (int64_t(1) << 31) - 512 || v >= (int64_t(1) << 31) - 512 || d > (1 << 24))
    return CCE_ERR_INVALID_ARGUMENT;
  if (dtype != CCE_DTYPE_BF16 && dtype != CCE_DTYPE_F16) return CCE_ERR_UNSUPPORTED_DTYPE;
  if (d_e == nullptr && d_c == nullptr && d_bias == nullptr) return CCE_OK;
  if (!aligned16(e) || !aligned16(c) || d % kDmaBK != 0 || stride_e % 8 != 0 || stride_cv % 8 != 0 || stride_cd != 1)
    return CCE_ERR_MISALIGNED;
  if (stride_e >= (int64_t(1) << 30) || stride_cv >= (int64_t(1) << 30)) return CCE_ERR_INVALID_ARGUMENT;
  if ((d_e != nullptr && !aligned16(d_e)) || (d_c != nullptr && !aligned16(d_c))) return CCE_ERR_MISALIGNED;
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0)
    return workspace == nullptr ? CCE_ERR_WORKSPACE_TOO_SMALL : CCE_ERR_MISALIGNED;

  // ---- plan: [16-bit compensation term of the gradient that is carried][dz buffer] ------------------------------
  const bool split_de = (d_e != nullptr) && !d_e_is_fp32;
  // (the walk by rows needs the caller to have sized the workspace for it: a 16-bit d_e is what the size query's
  // flag says, and a d_c in fp32 beside it is added to in place)
  const bool by_rows = dense_walks_by_rows(b, v, split_de);
  const int64_t comp_bytes = dense_plan(b, v, d, split_de, 0).fixed_bytes;
  // the plan the size query made (both gradients wanted), so that its answer always suffices
  const DensePlan plan = dense_plan(b, v, d, split_de, workspace_bytes - comp_bytes);
  if (plan.unit == 0) return CCE_ERR_WORKSPACE_TOO_SMALL;
  uint16_t* dz = reinterpret_cast<uint16_t*>(static_cast<unsigned char*>(workspace) + comp_bytes);
  const int64_t vc = by_rows ? (v + 255) / 256 * 256 : plan.unit;
  const int64_t ldz = vc;

  ProductParams p;
  p.dz = dz;
  p.ldz = ldz;
  p.stride_cv = stride_cv;
  p.e = static_cast<const uint16_t*>(e);
  p.stride_e = stride_e;
  p.valids = valids;
  p.de_f32 = split_de ? nullptr : static_cast<float*>(d_e);
  p.de_hi = split_de ? static_cast<uint16_t*>(d_e) : nullptr;
  p.de_lo = (split_de && !by_rows) ? static_cast<uint16_t*>(workspace) : nullptr;
  p.ld_de = stride_e;
  p.dc_fp32 = d_c_is_fp32;
  p.ld_dc = stride_cv;
  p.dc_accumulate = 0;
  p.dc_lo = nullptr;
  p.dc_first = 1;
  p.de_rows_by_number = 0;
  p.b = b;
  p.d = static_cast<int>(d);

  using TileB = Tile4<BF16, true, true>;
  const int lds = TileB::LDS_BYTES;
  const int tiles_n = static_cast<int>((d + 255) / 256);
  hipError_t err;
#define CCE_LAUNCH_PRODUCT(KERN, BLOCKS)                                                            \
  do {                                                                                              \
    auto kern = KERN;                                                                               \
    static LdsLimitOnce lds_limit;                                                            \
    err = lds_limit.set(kern, lds);                                        \
    if (err != hipSuccess) return status_from_hip(err);                                             \
    hipLaunchKernelGGL(kern, dim3(BLOCKS), dim3(kProdThreads), lds, stream, p);                     \
  } while (0)

  const size_t es = 2;
  if (by_rows) {
    // ---- blocks of rows, the whole vocabulary each ------------------------------------------------------------
    const int64_t rb = plan.unit;
    p.c = static_cast<const uint16_t*>(c);
    p.n_cls = static_cast<int>(v);
    p.first_chunk = 1;  // d_e of a block is complete with its launch
    p.tiles_n = tiles_n;
    p.d_c = d_c;
    p.dc_lo = (d_c != nullptr && !d_c_is_fp32) ? static_cast<uint16_t*>(workspace) : nullptr;
    p.dc_tiles = (d_c != nullptr) ? static_cast<int>((v + 255) / 256) * tiles_n : 0;
    p.dc_per_xcd = (p.dc_tiles + 7) / 8;
    for (int64_t r0 = 0; r0 < b; r0 += rb) {
      const int64_t n = (b - r0 < rb) ? (b - r0) : rb;
      // Rows are numbered through valids when there is one (absolute rows of e: only the list moves on); without
      // one the block is the rows [r0, r0 + n) of e, and everything indexed by row moves with it.
      const int64_t shift_rows = (valids == nullptr) ? r0 : 0;
      const unsigned char* e_blk = static_cast<const unsigned char*>(e) + shift_rows * stride_e * es;
      const int32_t* valids_blk = valids ? valids + r0 : nullptr;
      const float* d_out_blk = d_out_is_scalar ? d_out : d_out + shift_rows;
      const float* d_lse_blk = d_lse ? d_lse + shift_rows : nullptr;
      int st = dense_dz_launch(e_blk, c, bias, lse + r0, d_out_blk, d_out_is_scalar, d_lse_blk, valids_blk,
                               targets + shift_rows, dz, ldz, 0, 1, n_rows - shift_rows, n, v, d, stride_e, stride_cv,
                               stride_cd, grad_scale, shift, target_offset, softcap, dtype, stream);
      if (st != CCE_OK) return st;
      p.e = reinterpret_cast<const uint16_t*>(e_blk);
      p.valids = valids_blk;
      p.de_hi = static_cast<uint16_t*>(d_e) + shift_rows * stride_e;
      p.b = n;
      p.dc_first = (r0 == 0) ? 1 : 0;
      p.dc_accumulate = (r0 == 0) ? 0 : 1;  // an fp32 d_c is written by the first block and added to by the others
      p.de_tiles = static_cast<int>((n + 255) / 256) * tiles_n;
      p.de_per_xcd = (p.de_tiles + 7) / 8;
      p.de_first = (v > n) ? 1 : 0;
      const int blocks = (p.dc_per_xcd + p.de_per_xcd) * 8;
      if (dtype == CCE_DTYPE_BF16) CCE_LAUNCH_PRODUCT((dense_products_kernel<BF16, true>), blocks);
      else CCE_LAUNCH_PRODUCT((dense_products_kernel<F16, true>), blocks);
      if (d_bias != nullptr) {
        const unsigned cblocks = static_cast<unsigned>((v + 63) / 64);
        if (dtype == CCE_DTYPE_BF16)
          hipLaunchKernelGGL(dz_colsum_kernel<BF16>, dim3(cblocks), dim3(1024), 0, stream, dz, ldz, n, static_cast<int>(v),
                             d_bias);
        else
          hipLaunchKernelGGL(dz_colsum_kernel<F16>, dim3(cblocks), dim3(1024), 0, stream, dz, ldz, n, static_cast<int>(v),
                             d_bias);
      }
      err = hipGetLastError();
      if (err != hipSuccess) return status_from_hip(err);
    }
    return status_from_hip(hipGetLastError());
  }
  for (int64_t v0 = 0; v0 < v; v0 += vc) {
    const int64_t n = (v - v0 < vc) ? (v - v0) : vc;
    const unsigned char* c_chunk = static_cast<const unsigned char*>(c) + v0 * stride_cv * es;
    const void* bias_chunk = bias ? static_cast<const unsigned char*>(bias) + v0 * es : nullptr;
    int st = dense_dz_launch(e, c_chunk, bias_chunk, lse, d_out, d_out_is_scalar, d_lse, valids, targets, dz, ldz, 0, 1,
                             n_rows, b, n, d, stride_e, stride_cv, stride_cd, grad_scale, shift, target_offset + v0,
                             softcap, dtype, stream);
    if (st != CCE_OK) return st;
    p.c = reinterpret_cast<const uint16_t*>(c_chunk);
    p.n_cls = static_cast<int>(n);
    p.first_chunk = (v0 == 0) ? 1 : 0;
    p.tiles_n = tiles_n;
    p.d_c = nullptr;
    p.dc_tiles = 0;
    if (d_c != nullptr) {
      p.d_c = static_cast<unsigned char*>(d_c) + v0 * stride_cv * (d_c_is_fp32 ? 4 : 2);
      p.dc_tiles = static_cast<int>((n + 255) / 256) * tiles_n;
    }
    p.dc_per_xcd = (p.dc_tiles + 7) / 8;
    p.de_tiles = (d_e != nullptr) ? static_cast<int>((b + 255) / 256) * tiles_n : 0;
    p.de_per_xcd = (p.de_tiles + 7) / 8;
    p.de_first = (n > b) ? 1 : 0;
    const int blocks = (p.dc_per_xcd + p.de_per_xcd) * 8;
    if (blocks > 0) {
      if (dtype == CCE_DTYPE_BF16) {
        if (split_de) CCE_LAUNCH_PRODUCT((dense_products_kernel<BF16, true>), blocks);
        else CCE_LAUNCH_PRODUCT((dense_products_kernel<BF16, false>), blocks);
      } else {
        if (split_de) CCE_LAUNCH_PRODUCT((dense_products_kernel<F16, true>), blocks);
        else CCE_LAUNCH_PRODUCT((dense_products_kernel<F16, false>), blocks);
      }
    }
    if (d_bias != nullptr) {
      const unsigned blocks = static_cast<unsigned>((n + 63) / 64);
      if (dtype == CCE_DTYPE_BF16)
        hipLaunchKernelGGL(dz_colsum_kernel<BF16>, dim3(blocks), dim3(1024), 0, stream, dz, ldz, b, static_cast<int>(n),
                           d_bias + v0);
      else
        hipLaunchKernelGGL(dz_colsum_kernel<F16>, dim3(blocks), dim3(1024), 0, stream, dz, ldz, b, static_cast<int>(n),
                           d_bias + v0);
    }
    err = hipGetLastError();
    if (err != hipSuccess) return status_from_hip(err);
  }
#undef CCE_LAUNCH_PRODUCT

  return status_from_hip(hipGetLastError());
}

// ---- the two products of one chunk on their own ----------------------------------------------------------------
extern "C" int cce_backward_products(const void* dz, int64_t ldz, const void* c, int64_t stride_cv,
                                     const void* e, int64_t stride_e, const int32_t* valids,
                                     float* d_e, int64_t ld_de, float* d_c, int64_t ld_dc, int d_c_accumulate,
                                     int64_t b, int64_t n_cls, int64_t d, int dtype, void* stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (b < 0 || n_cls < 0 || d <= 0) return CCE_ERR_INVALID_ARGUMENT;
  if (b == 0 || n_cls == 0) return CCE_OK;
  if (dz == nullptr || (d_e != nullptr && c == nullptr) || (d_c != nullptr && e == nullptr)) return CCE_ERR_INVALID_ARGUMENT;
  if (dtype != CCE_DTYPE_BF16 && dtype != CCE_DTYPE_F16) return CCE_ERR_UNSUPPORTED_DTYPE;
  if (b >= (int64_t(1) << 31) - 512 || n_cls >= (int64_t(1) << 31) - 512 || d > (1 << 24)) return CCE_ERR_INVALID_ARGUMENT;
  if (ldz >= (int64_t(1) << 30) || stride_cv >= (int64_t(1) << 30) || stride_e >= (int64_t(1) << 30))
    return CCE_ERR_INVALID_ARGUMENT;
  if (d_e == nullptr && d_c == nullptr) return CCE_OK;
  if (!aligned16(dz) || ldz % 8 != 0 || ldz < (n_cls + 63) / 64 * 64 || d % 8 != 0) return CCE_ERR_MISALIGNED;
  if (d_e != nullptr && (!aligned16(c) || stride_cv % 8 != 0 || !aligned16(d_e) || ld_de % 4 != 0 || ld_de < d))
    return CCE_ERR_MISALIGNED;
  if (d_c != nullptr && (!aligned16(e) || stride_e % 8 != 0 || !aligned16(d_c) || ld_dc % 4 != 0 || ld_dc < d))
    return CCE_ERR_MISALIGNED;

  ProductParams p;
  p.dz = static_cast<const uint16_t*>(dz);
  p.ldz = ldz;
  p.c = static_cast<const uint16_t*>(c);
  p.stride_cv = stride_cv;
  p.e = static_cast<const uint16_t*>(e);
  p.stride_e = stride_e;
  p.valids = valids;
  p.de_f32 = d_e;
  p.de_hi = nullptr;
  p.de_lo = nullptr;
  p.ld_de = ld_de;
  p.de_rows_by_number = 1;
  p.first_chunk = 0;
  p.d_c = d_c;
  p.ld_dc = ld_dc;
  p.dc_fp32 = 1;
  p.dc_accumulate = d_c_accumulate;
  p.dc_lo = nullptr;
  p.dc_first = 1;
  p.b = b;
  p.d = static_cast<int>(d);
  p.n_cls = static_cast<int>(n_cls);
  p.tiles_n = static_cast<int>((d + 255) / 256);
  p.dc_tiles = (d_c != nullptr) ? static_cast<int>((n_cls + 255) / 256) * p.tiles_n : 0;
  p.de_tiles = (d_e != nullptr) ? static_cast<int>((b + 255) / 256) * p.tiles_n : 0;
  p.dc_per_xcd = (p.dc_tiles + 7) / 8;
  p.de_per_xcd = (p.de_tiles + 7) / 8;
  p.de_first = (n_cls > b) ? 1 : 0;
  const int blocks = (p.dc_per_xcd + p.de_per_xcd) * 8;
  const int lds = Tile4<BF16, true, true>::LDS_BYTES;
  hipError_t err;
  if (dtype == CCE_DTYPE_BF16) {
    auto kern = dense_products_kernel<BF16, false>;
    static LdsLimitOnce lds_limit;
        err = lds_limit.set(kern, lds);
    if (err != hipSuccess) return status_from_hip(err);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(kProdThreads), lds, stream, p);
  } else {
    auto kern = dense_products_kernel<F16, false>;
    static LdsLimitOnce lds_limit;
        err = lds_limit.set(kern, lds);
    if (err != hipSuccess) return status_from_hip(err);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(kProdThreads), lds, stream, p);
  }
  return status_from_hip(hipGetLastError());
}
