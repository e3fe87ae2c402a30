// Matrix transpose through a padded LDS tile: out[c*rows + r] = x[r*cols + c].
//
// A tile covers 256 input rows x 64 input columns.  It is read with streaming float4 loads
// along the input rows (256-byte pieces), staged in LDS (rows permuted and skewed so that neither side meets bank conflicts), and written
// with streaming float4 stores along the output rows: every output row of the tile receives 256
// consecutive floats, a full 1 KiB burst.  Workgroups are numbered down the input rows first, so
// that neighbouring workgroups extend each other's output bursts.  On MI355X the long write
// bursts matter more than the read side: this shape measures 6.1-6.2 TB/s on [16384 x 16384]
// against 4.1-5.4 TB/s for 64x64 and 128x128 tiles in either order.  Very tall matrices
// (rows >= 16 cols) walk the tiles in groups of 8 tile rows instead, so that the workgroups in
// flight also spread over the columns: [131072 x 1024] 4.5 -> 5.6 TB/s, [65536 x 2048] 4.7 -> 5.3;
// squarer and wide shapes measured up to 10 % slower that way and keep the plain order.
// Tall matrices of 2048, 3072 or 4096 columns (4 cols <= rows < 64 cols, output rows on 64-byte
// boundaries) and wide ones of 64, 128 or 192 rows take the mirrored tile, 64 input rows x 256 input
// columns (1 KiB read pieces, 256-byte write bursts), walked along the input rows' direction in
// groups of 8 tile columns: measured at 2^27 elements, [32768 x 4096] 4.85 -> 5.6 TB/s, [65536 x 2048]
// 5.25 -> 5.65, [128 x 2^20] 4.7 (chunk kernel) -> 5.9.  It pays where the input pitch is 8 or 16 KiB;
// other widths, squarer and wide shapes are 5-25 % slower with it ([16384 x 16384] 5.7 against 6.2,
// [30000 x 4000] 4.3 against 5.4).
// 8 B/element of HBM traffic, the algorithmic minimum.  beta selects `=` (0) or `+=` (1).
#include "common.hpp"

namespace slhip {

// TR input rows (= floats per output burst) by TC input columns per tile.  COLS_FIRST: tiles are
// walked in groups of `group` tile columns, column index fastest; else in groups of `group` tile
// rows, row index fastest.
template <int TR, int TC, bool COLS_FIRST, bool VEC_LD, bool VEC_ST, bool ACC>
__global__ __launch_bounds__(256) void transpose_kernel(size_t rows, size_t cols, const float* __restrict__ x,
                                                        float* out, unsigned tiles_r, unsigned group) {
  // Tile element (r, c) lives at ((r % 4) * 64 + r / 4) * 65 + c + 17 * (r % 4).  The store side of
  // the kernel has lane l fetch rows 4l .. 4l+3 of one column: with plain [r][c] rows, whatever the
  // pitch, lanes 8 apart meet on the same bank (four to a bank); here lane l's four rows sit 65 words
  // from lane l+1's, one bank further on.  The 17 * (r % 4) skew keeps the load side, where a wave
  // writes four consecutive rows at a time (vector form) or 64 (scalar form reads them back), on
  // distinct banks as well.
  __shared__ float tile_mem[TR * (TC + 1) + 52];
  auto tile = [&](int r, int c) -> float& { return tile_mem[((r & 3) * (TR / 4) + (r >> 2)) * (TC + 1) + c + 17 * (r & 3)]; };
  // (group = tiles_r, rows first: straight down the rows, column by column)
  const unsigned tiles_c = gridDim.x / tiles_r;
  const unsigned tiles_fast = COLS_FIRST ? tiles_c : tiles_r, tiles_slow = COLS_FIRST ? tiles_r : tiles_c;
  const unsigned in_group = group * tiles_slow;
  const unsigned first = blockIdx.x / in_group * group;
  const unsigned gsize = tiles_fast - first < group ? tiles_fast - first : group;
  const unsigned local = blockIdx.x % in_group;
  const size_t t_fast = first + local % gsize, t_slow = local / gsize;
  const size_t tr = COLS_FIRST ? t_slow : t_fast, tc = COLS_FIRST ? t_fast : t_slow;
  const size_t r0 = tr * TR, c0 = tc * TC;
  const int t = threadIdx.x;

  if (VEC_LD) {
    constexpr int LPR = TC / 4, RPP = 256 / LPR, NP = TR / RPP;  // float4 per tile row, rows per pass, passes
    const int lx = t % LPR, ly = t / LPR;
    // All loads of a thread (16) are issued before the first LDS store: only two tiles fit a CU,
    // so the bytes in flight have to come from each thread (64 VGPRs), not from occupancy.
    float4 v[NP];
    const bool full = r0 + TR <= rows && c0 + TC <= cols;
    if (full) {
#pragma unroll
      for (int p = 0; p < NP; ++p) v[p] = ld4s(x + (r0 + ly + RPP * p) * cols + c0 + 4 * lx);
    } else {
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const size_t r = r0 + ly + RPP * p, c = c0 + 4 * lx;
        if (r >= rows || c >= cols) {
          v[p] = make_float4(0.f, 0.f, 0.f, 0.f);
        } else if (c + 3 < cols) {
          v[p] = ld4s(x + r * cols + c);
        } else {  // the vector that straddles the end of a row of odd length
          const float* xr = x + r * cols;
          v[p] = make_float4(xr[c], c + 1 < cols ? xr[c + 1] : 0.f, c + 2 < cols ? xr[c + 2] : 0.f, 0.f);
        }
      }
    }
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int rr = ly + RPP * p;
      tile(rr, 4 * lx + 0) = v[p].x;
      tile(rr, 4 * lx + 1) = v[p].y;
      tile(rr, 4 * lx + 2) = v[p].z;
      tile(rr, 4 * lx + 3) = v[p].w;
    }
  } else {
    static_assert(VEC_LD || TC == 64, "the scalar load side is written for 64 columns");
    const int lx = t & 63, ly = t >> 6;  // 64 columns, 4 rows per pass
#pragma unroll 4
    for (int p = 0; p < TR / 4; ++p) {
      const int rr = ly + 4 * p;
      const size_t r = r0 + rr, c = c0 + lx;
      tile(rr, lx) = (r < rows && c < cols) ? x[r * cols + c] : 0.0f;
    }
  }
  __syncthreads();
  if (VEC_ST) {
    constexpr int LPR = TR / 4, RPP = 256 / LPR, NP = TC / RPP;  // float4 per output row of the tile, output rows per pass
    const int lx = t % LPR, ly = t / LPR;
    // Sixteen lanes cover an output row of the 64-row tile, so a wave reads four columns of the tile at
    // a time.  Side by side they share LDS banks four ways; sixteen apart they do not, which pays when
    // the output rows are short and lie close together anyway ([128 x 2^20] 5.74 -> 5.95 TB/s) and costs
    // when they are long: the wave's four stores then land 16 output rows apart ([32768 x 4096],
    // output rows of 128 KiB: 5.63 -> 5.40)
    const bool spread = TR == 64 && rows <= 512;
    const size_t orow0 = r0 + 4 * lx;
    // `+=`: all reads of the old output before the first store (a read after a store to what may be
    // the same memory waits for that store)
    float4 old[NP];
    if (ACC) {
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const size_t oc = c0 + (spread ? ly * NP + p : ly + RPP * p);
        old[p] = (oc < cols && orow0 + 3 < rows) ? ld4s(out + oc * rows + orow0) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int cc = spread ? ly * NP + p : ly + RPP * p;  // input column = output row
      const size_t oc = c0 + cc;
      if (oc < cols && orow0 < rows) {
        float4 v = make_float4(tile(4 * lx + 0, cc), tile(4 * lx + 1, cc), tile(4 * lx + 2, cc), tile(4 * lx + 3, cc));
        float* p_out = out + oc * rows + orow0;
        if (orow0 + 3 < rows) {
          if (ACC) { v.x += old[p].x; v.y += old[p].y; v.z += old[p].z; v.w += old[p].w; }
          st4s(p_out, v);
        } else {  // the vector that straddles the end of an output row of odd length
          if (orow0 < rows) p_out[0] = ACC ? p_out[0] + v.x : v.x;
          if (orow0 + 1 < rows) p_out[1] = ACC ? p_out[1] + v.y : v.y;
          if (orow0 + 2 < rows) p_out[2] = ACC ? p_out[2] + v.z : v.z;
        }
      }
    }
  } else {
    static_assert(VEC_ST || TR == 256, "the scalar store side is written for 256 rows");
#pragma unroll 4
    for (int p = 0; p < TC; ++p) {  // one output row per pass, 256 consecutive floats
      const size_t oc = c0 + p, orow = r0 + t;
      if (oc < cols && orow < rows) {
        float v = tile(t, p);
        float* p_out = out + oc * rows + orow;
        if (ACC) v += *p_out;
        *p_out = v;
      }
    }
  }
}

// The tile (TR x TC = 256 x 64 or 128 x 128) for matrices whose output rows do not start on 64-byte
// boundaries (rows not a multiple of 16, or an output that starts off the grid).  What a tile writes of
// output row c is then not the floats [r0, r0 + TR) but the piece [r0 - d_c, r0 + TR - d_c), d_c < 16 chosen per
// output row so that the piece starts and ends on 64-byte boundaries of the output: a 64-byte block
// that two tiles each write a part of reaches the memory as two partial writes (see the chunk kernel
// below, which does the same), and every vector store is aligned.  The tile stages 16 rows more than
// it writes, which the tile above it stages too.  The pieces at the two ends of an output row are
// cut there; what lies before a piece's first aligned vector and behind its last whole one goes
// float by float, thread c for output row c.  Same LDS layout as above: lane l of a wave fetches
// the rows s + 4 l .. s + 4 l + 3 of one column, whatever s, and meets no bank twice.
// [13421 x 10000] 3.9 -> 4.7 TB/s, [65521 x 2048] 4.45 -> 5.15, [134217 x 1000] 4.1 -> 4.6, [16383 x 16385]
// 4.1 -> 4.5, [12345 x 6789] 3.95 -> 4.2 with the 256 x 64 tile (the host's choice between the two tiles and the
// plain one is described where it is made).  (Without the unconditional loads of a whole tile - the
// `full` path - the same kernel measured 3-12 % behind the plain tile on every shape.)
template <bool ACC, int TR, int TC>
__global__ __launch_bounds__(256) void transpose_shift_kernel(size_t rows, size_t cols, const float* __restrict__ x,
                                                              float* out, unsigned tiles_r, unsigned group) {
  constexpr int H = 16, LR = TR + H;
  static_assert(TR % 64 == 0 && TC % 64 == 0 && LR % (1024 / TC) == 0 && TC <= 256, "tile shape");
  __shared__ float tile_mem[LR * (TC + 1) + 52];
  auto tile = [&](int r, int c) -> float& { return tile_mem[((r & 3) * (LR / 4) + (r >> 2)) * (TC + 1) + c + 17 * (r & 3)]; };
  const unsigned tiles_c = gridDim.x / tiles_r;
  const unsigned in_group = group * tiles_c;
  const unsigned first = blockIdx.x / in_group * group;
  const unsigned gsize = tiles_r - first < group ? tiles_r - first : group;
  const unsigned local = blockIdx.x % in_group;
  const size_t tr = first + local % gsize, tc = local / gsize;
  const size_t r0 = tr * TR, c0 = tc * TC;
  const size_t rb = r0 >= H ? r0 - H : 0;  // the first staged row: the first tile row has nothing above it
  const int staged = (int)(r0 - rb) + TR;  // rows rb .. rb + staged - 1, as far as the matrix goes
  const int t = threadIdx.x;
  {
    constexpr int LPR = TC / 4, RPP = 256 / LPR, NP = LR / RPP;  // float4 per tile row, rows per pass, passes
    const int lx = t % LPR, ly = t / LPR;
    float4 v[NP];
    const bool full = staged == LR && rb + LR <= rows && c0 + TC <= cols;
    if (full) {
#pragma unroll
      for (int p = 0; p < NP; ++p) v[p] = ld4s(x + (rb + ly + RPP * p) * cols + c0 + 4 * lx);
    } else {
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const int rr = ly + RPP * p;
        const size_t r = rb + rr, c = c0 + 4 * lx;
        if (rr >= staged || r >= rows || c >= cols) {
          v[p] = make_float4(0.f, 0.f, 0.f, 0.f);
        } else if (c + 3 < cols) {
          v[p] = ld4s(x + r * cols + c);
        } else {
          const float* xr = x + r * cols;
          v[p] = make_float4(xr[c], c + 1 < cols ? xr[c + 1] : 0.f, c + 2 < cols ? xr[c + 2] : 0.f, 0.f);
        }
      }
    }
    // a row of more than 16 vectors per wave instruction: lanes 8 apart would meet on a bank with the
    // same component, so lane lx stores component (j + lx / 8) % 4 in the j-th instruction
    const int rot = LPR > 16 ? (lx >> 3) & 3 : 0;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int rr = ly + RPP * p;
      if (LPR > 16) {
        const float e[4] = {v[p].x, v[p].y, v[p].z, v[p].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int q = (j + rot) & 3;
          tile(rr, 4 * lx + q) = q == 0 ? e[0] : q == 1 ? e[1] : q == 2 ? e[2] : e[3];
        }
      } else {
        tile(rr, 4 * lx + 0) = v[p].x;
        tile(rr, 4 * lx + 1) = v[p].y;
        tile(rr, 4 * lx + 2) = v[p].z;
        tile(rr, 4 * lx + 3) = v[p].w;
      }
    }
  }
  __syncthreads();
  constexpr int LPO = TR / 4, OPP = 256 / LPO, NP = TC / OPP;  // lanes per output row, output rows per pass, passes
  const int lx = t % LPO, ly = t / LPO;
  // the output row of pass p: with 16 lanes per output row a wave takes the rows {j, j + 16, j + 1, j + 17} of
  // a block of 32 (lane l reads LDS bank l + the row's number: two rows 16 apart fill the 32 banks)
  auto out_row = [&](int p) {
    if (LPO >= 32) return ly + OPP * p;
    const int q = p * 4 + (t >> 6), g = (t >> 4) & 3;
    return (q >> 3) * 32 + 2 * (q & 7) + (g >> 1) + 16 * (g & 1);
  };
  // everything in rows relative to the first staged one, in 32 bits
  const int off = (int)(r0 - rb);  // H, or 0 in the first tile row
  const int nst = rows - rb < (size_t)staged ? (int)(rows - rb) : staged;
  const int ob = (int)((reinterpret_cast<uintptr_t>(out) >> 2) & (H - 1)), lm = (int)(rows & (H - 1));
  // the piece of output row c0 + cc: staged rows [lo, hi); returns the floats before its first aligned vector
  auto piece = [&](int cc, int& lo, int& hi) {
    const int d = (ob + (int)((c0 + cc) & (H - 1)) * lm) & (H - 1);  // (r0 is a multiple of 64)
    lo = off > d ? off - d : 0;
    hi = off + TR - d < nst ? off + TR - d : nst;
    return lo ? 0 : (4 - (d & 3)) & 3;  // lo > 0: the piece starts on a 64-byte boundary
  };
  float* const obeg = out + rb;
  float4 old[NP];
  if (ACC) {
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int cc = out_row(p);
      int lo, hi;
      const int l = piece(cc, lo, hi) + lo + 4 * lx;
      old[p] = (c0 + cc < cols && l + 3 < hi) ? ld4s(obeg + (c0 + cc) * rows + l) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int cc = out_row(p);
    int lo, hi;
    const int l = piece(cc, lo, hi) + lo + 4 * lx;
    if (c0 + cc < cols && l + 3 < hi) {
      float4 v = make_float4(tile(l, cc), tile(l + 1, cc), tile(l + 2, cc), tile(l + 3, cc));
      if (ACC) { v.x += old[p].x; v.y += old[p].y; v.z += old[p].z; v.w += old[p].w; }
      st4s(obeg + (c0 + cc) * rows + l, v);
    }
  }
  // at most three floats before and three behind the vectors of a piece: thread c sees to output row c
  if (t < TC && c0 + t < cols) {
    int lo, hi;
    int lead = piece(t, lo, hi) + lo;
    if (lo < hi) {
      if (lead > hi) lead = hi;
      const int tail = lead + ((hi - lead) & ~3);
      float* orow = obeg + (c0 + t) * rows;
      for (int l = lo; l < lead; ++l) orow[l] = ACC ? orow[l] + tile(l, t) : tile(l, t);
      for (int l = tail; l < hi; ++l) orow[l] = ACC ? orow[l] + tile(l, t) : tile(l, t);
    }
  }
}

// Matrices with few columns (or few rows): the tile above would be mostly empty.  A chunk of R whole
// rows of the narrow matrix is one contiguous run of R*S floats (S = the short side) on the narrow
// side and S runs of R floats on the other.  A workgroup moves one such chunk through LDS: both
// sides are read and written with consecutive lanes on consecutive floats.  NARROW_IN: the input
// is the narrow matrix [long x S]; else the input is [S x long] and the output is narrow.
// The LDS index is skewed by one word per 32 (a power-of-two S would pile a column onto one bank).
// CHUNK floats per workgroup of NTH threads.  64 KiB chunks on 512 threads serve narrow inputs up
// to 56 columns and narrow outputs up to 200 rows (against 32 KiB the runs on the wide side are twice
// as long: narrow inputs of 10..56 columns gain 5-11 %, narrow outputs of 100..200 rows 5-11 %);
// 128 KiB chunks on 1024 threads, one workgroup to a CU, serve tall inputs of 57..256 columns that are
// not a multiple of 64 wide, where the runs of a 64 KiB chunk on the wide side are too short
// ([1342177 x 100]: 3.7 TB/s with 64 KiB chunks, 3.4 for the tiled kernel, whose last tile column is
// mostly empty) - unless the output runs start on 64-byte boundaries by themselves, where 64 KiB
// chunks are ahead up to 200 columns ([1342176 x 100] 5.5 against 5.3).
// What a chunk writes of an output run is a piece that starts on a 64- or 128-byte boundary of the
// output and is a multiple of that long: a piece that ends inside such a block leaves the block to
// two workgroups on two L2s, and the memory sees two partial writes ([1342176 x 100], whose runs
// start on 128-byte boundaries: 5.4 TB/s; [1342180 x 100]: 4.0-4.4 with the same code).  With an odd
// long side the boundaries lie elsewhere in every run, so the chunk shifts its piece of run s by
// d_s floats and stages 16 or 32 more rows of the input than it writes ([1342177 x 100] 4.7 -> 5.05
// TB/s, [13421772 x 10] 5.2 -> 5.7, [4067000 x 33] 5.0 -> 5.5, [958698 x 140] 4.4 -> 5.0).
// Stores are streaming (non-temporal): 4-20 % over plain stores on every shape measured
// ([100 x 1342177] 4.3 -> 5.2 TB/s, [13421772 x 10] 5.0 -> 5.2, [33 x 4067000] 5.5 -> 5.9).
__device__ __forceinline__ int ts_skew(int i) { return i + (i >> 5); }
template <bool NARROW_IN, bool ACC, int CHUNK, int NTH>
__global__ __launch_bounds__(NTH) void transpose_narrow_kernel(size_t long_side, int S, int R, const float* __restrict__ x,
                                                               float* out, unsigned chunks, int halo, int align) {
  __shared__ float buf[CHUNK + CHUNK / 32 + 4];
  // LDS holds the chunk in the narrow matrix's order: element (l, s) at l*S + s.  Global memory is
  // touched with dword-aligned float4 on both sides (scalar accesses stream at a third of the rate).
  // Every vector of a chunk is requested before the first one is stored to LDS: a loop that loads
  // and stores in turn keeps one request per thread in flight.
  // A workgroup takes chunks blockIdx.x, blockIdx.x + gridDim.x, ...: the vectors of its next chunk
  // are requested before the current one is written out, so a CU that holds a single workgroup
  // (128 KiB chunks) still has loads in flight while it stores.
  constexpr int NJ = CHUNK / (4 * NTH);
  const int RV = R >> 2;  // vectors per run on the wide side (R is a multiple of 4 whenever a run has vectors)
  float4 v[NJ];
  // NARROW_IN with halo = align (16 or 32 floats; the runs of the output do not all start on
  // boundaries of that many floats): chunk c writes, of output run s, the floats
  // [c R - d_s, c R + R - d_s) (cut to the run), where d_s < align is what puts that piece on such a
  // boundary of the output; it stages the rows [c R - halo, c R + R) of the input, `halo` rows of
  // which its neighbour stages too.
  // Otherwise (halo = 0): chunk c is the floats [c R, c R + R) of every run.
  auto first_row = [&](unsigned c) { const size_t l0 = (size_t)c * R; return NARROW_IN && c ? l0 - halo : l0; };
  auto rows_of = [&](unsigned c) {
    const size_t l0 = (size_t)c * R, lb = first_row(c);
    if (lb >= long_side) return 0;
    return l0 + R <= long_side ? (int)(l0 + R - lb) : (int)(long_side - lb);
  };
  auto request = [&](unsigned c) {
    const size_t l0 = first_row(c);
    const int nr = rows_of(c);
    if (NARROW_IN) {
      const float* src = x + l0 * S;
      const int len4 = (nr * S) & ~3;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int i = 4 * threadIdx.x + 4 * NTH * j;
        if (i < len4) v[j] = ld4s(src + i);
      }
    } else {
      // the S runs of nr floats, cut into vectors and dealt out over the threads: vector k of the
      // chunk is vector k % RV of run k / RV
      const int nrv = nr >> 2;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int k = threadIdx.x + NTH * j, run = k / RV, lv = k - run * RV;
        if (run < S && lv < nrv) v[j] = ld4s(x + (size_t)run * long_side + l0 + 4 * lv);
      }
    }
  };
  auto stage = [&](unsigned c) {  // v, and the few floats beside the vectors, into LDS
    const size_t l0 = first_row(c);
    const int nr = rows_of(c), len = nr * S, nr4 = nr & ~3, len4 = len & ~3;
    if (NARROW_IN) {
      const float* src = x + l0 * S;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int i = 4 * threadIdx.x + 4 * NTH * j;
        if (i < len4) {
          buf[ts_skew(i)] = v[j].x; buf[ts_skew(i + 1)] = v[j].y; buf[ts_skew(i + 2)] = v[j].z; buf[ts_skew(i + 3)] = v[j].w;
        }
      }
      for (int i = len4 + threadIdx.x; i < len; i += NTH) buf[ts_skew(i)] = src[i];
    } else {
      const int nrv = nr4 >> 2;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int k = threadIdx.x + NTH * j, run = k / RV, lv = k - run * RV;
        if (run < S && lv < nrv) {
          const int l = 4 * lv;
          buf[ts_skew(l * S + run)] = v[j].x; buf[ts_skew((l + 1) * S + run)] = v[j].y;
          buf[ts_skew((l + 2) * S + run)] = v[j].z; buf[ts_skew((l + 3) * S + run)] = v[j].w;
        }
      }
      for (int s = 0; s < S; ++s) {
        const float* src = x + (size_t)s * long_side + l0;
        for (int l = nr4 + threadIdx.x; l < nr; l += NTH) buf[ts_skew(l * S + s)] = src[l];
      }
    }
  };
  auto drain = [&](unsigned c) {  // LDS to the output
    const size_t l0 = (size_t)c * R;
    const int nr = rows_of(c), len = nr * S, len4 = len & ~3;
    if (NARROW_IN) {
      // The S output runs, cut into vectors and dealt out over the threads as on the load side of
      // the other direction.  Run s starts at float s * long_side of the output, which is aligned
      // only by chance when the long side is odd; shifted by d_s, this chunk's piece of it starts
      // on a 64-byte boundary and is R floats long, so it is written as whole 64-byte blocks
      // (pieces that end inside a block leave it to two workgroups, which costs a sixth of the rate:
      // [1342177 x 100] 4.7 -> 5.2 TB/s).  The pieces at the two ends of a run are cut there: what
      // lies before the first aligned vector and behind the last whole one goes float by float.
      // (all of it in row numbers relative to the first staged row, in 32 bits)
      const size_t lb = first_row(c);
      const int off = (int)(l0 - lb);  // halo, or 0 for the first chunk
      const int ob = (int)((reinterpret_cast<uintptr_t>(out) >> 2) & (align - 1)), lm = (int)(long_side & (align - 1));
      // the piece of `run`: rows [lo, hi) of the staged ones; returns the floats before its first aligned vector
      auto piece = [&](int run, int& lo, int& hi) {
        const int d = (ob + run * lm) & (align - 1);
        lo = off > d ? off - d : 0;
        hi = off + R - d < nr ? off + R - d : nr;
        return lo ? 0 : (4 - (d & 3)) & 3;  // lo > 0: the piece starts on a boundary
      };
      float* const obeg = out + lb;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int k = threadIdx.x + NTH * j, run = k / RV, lv = k - run * RV;
        if (run < S) {
          int lo, hi;
          const int l = piece(run, lo, hi) + lo + 4 * lv;
          if (l + 3 < hi) {
            float* dst = obeg + (size_t)run * long_side + l;
            const int at = l * S + run;
            float4 w = make_float4(buf[ts_skew(at)], buf[ts_skew(at + S)], buf[ts_skew(at + 2 * S)], buf[ts_skew(at + 3 * S)]);
            if (ACC) { const float4 o = ld4(dst); w.x += o.x; w.y += o.y; w.z += o.z; w.w += o.w; }
            st4s(dst, w);
          }
        }
      }
      // at most three floats before and three behind the vectors of a piece (more when it holds no
      // whole vector): thread s sees to run s
      for (int run = threadIdx.x; run < S; run += NTH) {
        int lo, hi;
        int lead = piece(run, lo, hi) + lo;
        if (lo >= hi) continue;
        if (lead > hi) lead = hi;
        const int tail = lead + ((hi - lead) & ~3);
        float* dst = obeg + (size_t)run * long_side;
        for (int l = lo; l < lead; ++l) { const float t = buf[ts_skew(l * S + run)]; dst[l] = ACC ? dst[l] + t : t; }
        for (int l = tail; l < hi; ++l) { const float t = buf[ts_skew(l * S + run)]; dst[l] = ACC ? dst[l] + t : t; }
      }
    } else {
      float* dst = out + l0 * S;
      for (int i = 4 * threadIdx.x; i < len4; i += 4 * NTH) {
        float4 w = make_float4(buf[ts_skew(i)], buf[ts_skew(i + 1)], buf[ts_skew(i + 2)], buf[ts_skew(i + 3)]);
        if (ACC) { const float4 o = ld4g(dst + i); w.x += o.x; w.y += o.y; w.z += o.z; w.w += o.w; }
        st4s(dst + i, w);
      }
      for (int i = len4 + threadIdx.x; i < len; i += NTH) dst[i] = ACC ? dst[i] + buf[ts_skew(i)] : buf[ts_skew(i)];
    }
  };
  unsigned c = blockIdx.x;
  if (c >= chunks) return;
  request(c);
  for (; c < chunks; c += gridDim.x) {
    stage(c);
    __syncthreads();
    if (c + gridDim.x < chunks) request(c + gridDim.x);
    drain(c);
    __syncthreads();  // the next chunk's stage overwrites what this drain reads
  }
}

__global__ __launch_bounds__(64) void axpy_copy_kernel(size_t n, const float* __restrict__ x, float* out) {
  const size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (i < n) out[i] += x[i];
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_transpose(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out, float beta) {
  size_t len;
  SLHIP_REQUIRE(ctx && x && out, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  SLHIP_REQUIRE(beta == 0.0f || beta == 1.0f, "beta must be 0 (set) or 1 (accumulate)");
  if (x < out + len && out < x + len) {  // the same buffer, or any partial overlap
    set_error("slhip_transpose: out overlaps x (in-place transpose is not supported)");
    return SLHIP_EALIAS;
  }
  const bool acc = beta != 0.0f;
  if (rows == 1 || cols == 1) {  // a vector: the transpose is the same sequence of values
    if (!acc) return slhip_memcpy_d2d(ctx, out, x, len * sizeof(float));
    SLHIP_REQUIRE((len + 63) / 64 <= 0x7fffffffu, "vector too long for one launch");
    hipLaunchKernelGGL(axpy_copy_kernel, dim3((unsigned)((len + 63) / 64)), dim3(64), 0, ctx->stream, len, x, out);
    return post_launch();
  }
  // Which kernel (measured at 2^27 elements, TB/s, chunk kernel / 256 x 64 tiles): a narrow input
  // [long x S] with an odd long side: S = 33: 5.5 / 2.4, 56: 5.5 / 3.5, 64: 5.3 / 5.8, 72: 5.4 / -,
  // 100: 5.05 / 3.4, 128: 5.4 / 5.8, 140: 5.0 / -, 180: 4.9 / -, 200: 4.8 / 3.8, 250: 4.75 / -; a narrow output, input [S x long]: S = 48: 4.9 / 2.7, 64: 5.4 / 3.3, 100: 5.2 / 3.4,
  // 128: 5.8 / 4.1 (64 x 256 tiles: 5.9), 160: 4.4 / 4.0, 200: 4.9 / -, 224: 3.1 / -, 257: 2.6 / 3.4.
  const bool mirrored_rows = rows % 64 == 0 && rows >= 64 && rows <= 192 && cols >= 4 * rows;  // the 64 x 256 tile below
  // The pieces of the output runs that a narrow input's chunks write start on boundaries of `unit`
  // floats: 64 bytes, which is what the rate depends on ([1342176 / 1342160 / 1342168 / 1342180 x 100]:
  // runs that start on multiples of 128 / 64 / 32 / 16 bytes, 5.4 / 5.25 / 4.4 / 4.0 TB/s), or 128 where
  // that is free (the runs start there by themselves) or cheap (chunks of 256 rows and more: 1-5 %
  // faster again).  Odd long sides get there with a halo of that many rows.
  const int unit = cols <= 64 || (rows % 32 == 0 && (reinterpret_cast<uintptr_t>(out) & 127) == 0) ? 32 : 16;
  const bool runs_aligned = rows % unit == 0 && (reinterpret_cast<uintptr_t>(out) & (4 * unit - 1)) == 0;
  const bool narrow_in_wide = cols > 56 && cols <= 256 && cols % 64 != 0 && rows >= 16 * cols;
  const bool narrow_in_big = narrow_in_wide && !(runs_aligned && cols <= 200);
  const bool narrow_in = !narrow_in_big && (narrow_in_wide || (cols <= 56 && cols <= rows));
  const bool narrow_out = !narrow_in && !narrow_in_big && !mirrored_rows && rows <= 200 && rows < cols;
  if (narrow_in || narrow_in_big || narrow_out) {
    const bool in = !narrow_out;
    const size_t long_side = in ? rows : cols;
    const int S = (int)(in ? cols : rows);
    const int halo = in && !runs_aligned ? unit : 0;
    const int chunk = narrow_in_big ? 32768 : 16384;
    int R = chunk / S;
    if (in) R = (R - halo) & ~(unit - 1);  // the chunk holds `halo` rows more than it writes of every run
    else if (R >= 256) R &= ~31;  // runs that start on 128-byte boundaries of their rows, where that costs little
    else if (R >= 4) R &= ~3;  // whole vectors per run
    // (with a halo the last chunk ends unit - 1 floats or more behind the runs: every shifted piece ends inside it)
    const size_t blocks = (long_side + (halo ? halo - 1 : 0) + R - 1) / R;
    SLHIP_REQUIRE(blocks <= 0x7fffffffu, "matrix too large for one launch");
    // 128 KiB chunks: one workgroup per CU, each walking its share of the chunks; 64 KiB chunks: one
    // workgroup per chunk
    const size_t wgs = narrow_in_big && blocks > (size_t)ctx->num_cu ? (size_t)ctx->num_cu : blocks;
#define SL_TN(NI, A, CH, NT_) \
  hipLaunchKernelGGL((transpose_narrow_kernel<NI, A, CH, NT_>), dim3((unsigned)wgs), dim3(NT_), 0, ctx->stream, long_side, S, R, x, out, (unsigned)blocks, halo, unit)
    if (narrow_in_big) { if (acc) SL_TN(true, true, 32768, 1024); else SL_TN(true, false, 32768, 1024); }
    else if (in) { if (acc) SL_TN(true, true, 16384, 512); else SL_TN(true, false, 16384, 512); }
    else { if (acc) SL_TN(false, true, 16384, 512); else SL_TN(false, false, 16384, 512); }
#undef SL_TN
    return post_launch();
  }
  // The mirrored tile for wide matrices of 64, 128 or 192 rows and for tall ones of 2048, 3072 or 4096
  // columns whose output rows start on 64-byte boundaries (see the header).  It is a remedy for
  // input pitches of 8 and 16 KiB, where the 256 x 64 tile reads 256 pieces of 256 bytes that far
  // apart ([32768 x 4096] 4.85 -> 5.64 TB/s, [65536 x 2048] 5.23 -> 5.68, [16384 x 2048] 4.6 -> 5.2);
  // at any other width, and with output rows of odd length, the 256 x 64 tile with its 1 KiB write
  // bursts is ahead ([30000 x 4000] 4.27 -> 5.38, [32768 x 4000] 4.66 -> 5.59, [30000 x 3840] 4.8 -> 5.7,
  // [50000 x 5120] 4.9 -> 5.6, [32768 x 8192] 5.4 -> 6.0, [65521 x 2048] 3.3 -> 4.5, [50001 x 2001] 2.6 -> 4.1).
  const bool mirrored_cols = rows >= 4 * cols && rows < 64 * cols && cols % 1024 == 0 && cols >= 2048 && cols <= 4096 && rows % 16 == 0;
  if (mirrored_rows || mirrored_cols) {  // (taller still: the 256 x 64 tile in groups of 8 tile rows measures 2-3 % faster)
    const size_t tiles_r = (rows + 63) / 64, tiles_c = (cols + 255) / 256;
    SLHIP_REQUIRE(tiles_r * tiles_c <= 0x7fffffffu, "matrix too large for one launch");
    const unsigned group = tiles_c < 8 ? (unsigned)tiles_c : 8u;
    if (acc) hipLaunchKernelGGL((transpose_kernel<64, 256, true, true, true, true>), dim3((unsigned)(tiles_r * tiles_c)), dim3(256), 0, ctx->stream, rows, cols, x, out, (unsigned)tiles_r, group);
    else hipLaunchKernelGGL((transpose_kernel<64, 256, true, true, true, false>), dim3((unsigned)(tiles_r * tiles_c)), dim3(256), 0, ctx->stream, rows, cols, x, out, (unsigned)tiles_r, group);
    return post_launch();
  }
  constexpr int TR = 256, TC = 64;
  // Output rows that start off the 64-byte grid: pieces shifted per output row.  The 256 x 64 tile for
  // output rows of 8192 floats and more, 2^24 elements and more and an input pitch that is a multiple of
  // 64 bytes ([65521 x 2048] 5.1 TB/s against 5.0 for the square tile, [16385 x 16384] 5.45 against 5.1);
  // the 128 x 128 tile for every other pitch and for shorter output rows (from 256 floats): its 512-byte
  // input pieces straddle one 128-byte line in four where 256-byte pieces straddle one in two, and its
  // output pieces leave short output rows more whole pieces between their cut ends (the 256 x 64 tile lost
  // to the plain one there).  Against the 256 x 64 tile, shifted: [12345 x 6789] 4.17 -> 4.46, [9001 x 50001]
  // 4.05 -> 4.51, [23171 x 23169] 4.34 -> 4.63; against the plain tile: [8191 x 16385] 3.8 -> 4.75, [1001 x 100003]
  // 3.4 -> 4.55, [300 x 400001] 3.4 -> 4.2, [6001 x 20000] 4.6 -> 5.2, [4026 x 32768] 4.2 -> 4.7, [5000 x 3001] 36 ->
  // 32 us.  With fewer than 256 square tiles (or fewer than 2^24 elements below 1024 columns) the plain
  // tile stays ([1025 x 1025] 8 against 12 us, [8193 x 1000] 23 against 25, [100001 x 257] 48 against 55).
  if (cols >= 64 && (rows % 16 != 0 || (reinterpret_cast<uintptr_t>(out) & 63) != 0)) {
    const bool big = len >= (size_t(1) << 24);
    // (below 1024 columns also where the last column of 128-wide tiles would be emptier than that of 64-wide
    // ones: [100001 x 257] 48 against 56 us)
    const bool narrower = cols < 1024 && (cols + 63) / 64 * 64 < (cols + 127) / 128 * 128;
    if (rows >= 8192 && big && (cols % 16 == 0 || narrower)) {
      const size_t tiles_r = (rows + 15 + TR - 1) / TR, tiles_c = (cols + TC - 1) / TC;  // the last piece of every output row ends inside the last tile row
      SLHIP_REQUIRE(tiles_r * tiles_c <= 0x7fffffffu, "matrix too large for one launch");
      const unsigned group = rows >= 16 * cols ? (tiles_r < 8 ? (unsigned)tiles_r : 8u) : (unsigned)tiles_r;
      if (acc) hipLaunchKernelGGL((transpose_shift_kernel<true, 256, 64>), dim3((unsigned)(tiles_r * tiles_c)), dim3(256), 0, ctx->stream, rows, cols, x, out, (unsigned)tiles_r, group);
      else hipLaunchKernelGGL((transpose_shift_kernel<false, 256, 64>), dim3((unsigned)(tiles_r * tiles_c)), dim3(256), 0, ctx->stream, rows, cols, x, out, (unsigned)tiles_r, group);
      return post_launch();
    }
    const size_t tiles_r = (rows + 15 + 127) / 128, tiles_c = (cols + 127) / 128;
    if (rows >= 256 && (cols >= 1024 ? tiles_r * tiles_c >= 256 : big)) {
      SLHIP_REQUIRE(tiles_r * tiles_c <= 0x7fffffffu, "matrix too large for one launch");
      const unsigned group = rows >= 16 * cols ? (tiles_r < 8 ? (unsigned)tiles_r : 8u) : (unsigned)tiles_r;
      if (acc) hipLaunchKernelGGL((transpose_shift_kernel<true, 128, 128>), dim3((unsigned)(tiles_r * tiles_c)), dim3(256), 0, ctx->stream, rows, cols, x, out, (unsigned)tiles_r, group);
      else hipLaunchKernelGGL((transpose_shift_kernel<false, 128, 128>), dim3((unsigned)(tiles_r * tiles_c)), dim3(256), 0, ctx->stream, rows, cols, x, out, (unsigned)tiles_r, group);
      return post_launch();
    }
  }
  const size_t tiles_r = (rows + TR - 1) / TR, tiles_c = (cols + TC - 1) / TC;
  SLHIP_REQUIRE(tiles_r * tiles_c <= 0x7fffffffu, "matrix too large for one launch");
  const unsigned grid = (unsigned)(tiles_r * tiles_c);
  // rows and columns of any length take the vector paths (dword-aligned float4); the scalar
  // variants remain for matrices narrower than one vector
  const unsigned group = rows >= 16 * cols ? (tiles_r < 8 ? (unsigned)tiles_r : 8u) : (unsigned)tiles_r;
  const bool vld = cols >= 4;
  const bool vst = rows >= 4;
#define SL_TR(L, S, A) \
  hipLaunchKernelGGL((transpose_kernel<256, 64, false, L, S, A>), dim3(grid), dim3(256), 0, ctx->stream, rows, cols, x, out, (unsigned)tiles_r, group)
  if (vld && vst) { if (acc) SL_TR(true, true, true); else SL_TR(true, true, false); }
  else if (vld) { if (acc) SL_TR(true, false, true); else SL_TR(true, false, false); }
  else if (vst) { if (acc) SL_TR(false, true, true); else SL_TR(false, true, false); }
  else { if (acc) SL_TR(false, false, true); else SL_TR(false, false, false); }
#undef SL_TR
  return post_launch();
}
