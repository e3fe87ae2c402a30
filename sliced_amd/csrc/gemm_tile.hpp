// The tile machinery of the f32 GEMM: argument block, global -> LDS staging, MFMA fragment reads,
// the software-pipelined k loop and the whole-tile workgroup body.  Shared by the plain kernel
// (gemm.hip) and the spread-tail kernel (gemm_spread.hip), which are separate translation units
// on purpose: the plain kernel's k loop gains or loses about 1.5 % with the code the compiler
// happens to place around it, and a kernel added to its file moved it.
//
// A workgroup is WGM x WGN waves (2 x 2 unless said otherwise); every wave owns WM x WN
// accumulators of 32 x 32, so the workgroup's tile of C is (32*WM*WGM) x (32*WN*WGN): 128 x 128
// for large products, 64 x 64 for products whose 128 x 128 grid would leave most of the chip idle,
// and 128 x 128 on eight waves (2 x 4, each 64 x 32) for grids that give a CU a single workgroup.
#pragma once
#include <type_traits>

#include "common.hpp"

namespace slhip {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128;
constexpr int GEMM_BK = 32;  // measured against 16: 3-10 % faster on every form at 2048^3 and above

// One operand tile: XT rows or columns of the operand (64 or 128) by BK of k, staged by NT threads.
template <int BK, int XT, int NT = 256>
struct Cfg {
  static constexpr int KC_PITCH = BK + 4;  // [x][k] layout, k contiguous
  // [k][x] layout, x contiguous: rows of exactly XT words, and element (k, x) sits at column
  // x ^ 32 when bit 2 of k is set (xc_index).  An MFMA fragment read takes k = 8g + 4h + t for
  // the lanes' halves h = 0, 1: the swizzle puts the two halves on different banks, where padding
  // the rows did before - but with rows of 128 words every fragment address of a k tile is the
  // lane's base plus a multiple of 64 words, which ds_read2st64_b32 takes as an immediate.  With
  // padded rows (pitch 132) the four k of a group needed a base register each, computed in the
  // loop: 9 vector adds per k tile, paid for in matrix-core time (A*B 135.3 -> 139.5 TFLOP/s
  // with the adds taken out).
  static constexpr int XC_PITCH = XT;
  static constexpr int STAGE_FLOATS = XT * KC_PITCH > BK * XC_PITCH ? XT * KC_PITCH : BK * XC_PITCH;
  static constexpr int NV = BK * XT / 4 / NT;  // float4 per thread per operand tile
};

__device__ __forceinline__ int xc_swizzle(int k) { return ((k >> 2) & 1) << 5; }

// The 32-wide block of rows (or columns) of the workgroup's tile that wave coordinate w (of WG
// along this side) owns as its i-th: blocks are dealt out to the waves in turn, so a wave's blocks
// lie 32 * WG apart - a multiple of 64 for the two-by-two grid, which the fragment addressing
// above relies on.
template <int WG>
__device__ __forceinline__ constexpr int block_of(int w, int i) { return 32 * (w + WG * i); }

struct GemmArgs {
  size_t M, N, K;
  const float* A;
  const float* B;
  float* C;
  float beta;
  const float* bias;  // may be null
  int relu;
  float* pre_act;     // may be null
  const float* mask;  // may be null; else the product is multiplied by (mask[idx] >= 0) before beta*C is added
  unsigned tiles_m, tiles_n;
  unsigned splits;    // > 1: write raw partial sums to `partial[z][M*N]`
  size_t k_chunk;     // multiple of BK
  float* partial;
  int a_vec, b_vec;   // the operand's leading dimension is a multiple of 4: rows split into whole float4 loads
  size_t m_fast;      // M when both operand bases are 16-byte aligned as well, else 0: no tile counts as interior
};

// Spread tail (gemm_spread_kernel): workgroups below `first` compute whole tiles;
// workgroup first + w computes k tiles [w*units, (w+1)*units) of the sequence "tile `first`, all
// its kt_total k tiles; tile first + 1, ..." (`total` long).  Kept out of GemmArgs: the plain
// kernel's code, and with it its speed, depends on the layout of its argument block.
struct SpreadArgs {
  unsigned first, units, total, kt_total;
};

constexpr size_t SPREAD_SLOT = (size_t)BM * BN;  // floats of one partial tile in the workspace

// Operand tile held in registers between the global load and the LDS store.
template <int BK, int XT, int NT = 256>
struct Frag {
  float4 v[Cfg<BK, XT, NT>::NV];
};

// How a k tile is fetched from global memory.
//   LOAD_FAST   the whole tile is inside the operand, float4-loadable and 16-byte aligned:
//               unconditional aligned float4 (the aligned type measures 2 % faster on A*B than the
//               dword-aligned one, although both become global_load_dwordx4)
//   LOAD_XCLAMP any operand, any alignment, but only k tiles that end before the operand's last k
//               index: dword-aligned float4 loads whose x coordinate is clamped into the operand and
//               nothing else.  Rows and columns outside the operand receive whatever the clamped
//               load returns - they only reach rows and columns of C that are never stored.  A
//               vector that straddles the end of a row of odd length reads on into the next row,
//               which exists because the tile stops short of the last k index.
//   LOAD_VCLAMP the operand is float4-loadable; any k tile (the k remainder in particular):
//               dword-aligned float4 loads from coordinates clamped in x and k, zeroed afterwards
//   LOAD_SCALAR anything else (the last k tiles of operands whose rows do not split into float4):
//               one load per element from clamped coordinates, zeroed afterwards
// No variant branches around a load, so all loads of a tile are in flight together (a version
// with one branch per element took about 15 us per k tile on tiny problems: each load waited for
// the one before it).
enum { LOAD_FAST = 0, LOAD_VCLAMP = 1, LOAD_SCALAR = 2, LOAD_XCLAMP = 3 };

// k-contiguous source: element (x, k) at src[x*ld + k]; tile XT x BK.
template <int BK, int XT, int MODE, int NT = 256>
__device__ __forceinline__ void load_kc(Frag<BK, XT, NT>& f, const float* __restrict__ src, size_t ld, size_t X, size_t Kend,
                                        size_t x0, size_t k0) {
  constexpr int VPR = BK / 4, RPP = NT / VPR;  // float4 per row, rows per pass
  const int kq = threadIdx.x % VPR, xr = threadIdx.x / VPR;
#pragma unroll
  for (int p = 0; p < Cfg<BK, XT, NT>::NV; ++p) {
    const size_t x = x0 + xr + RPP * p, k = k0 + 4 * kq;
    if (MODE == LOAD_FAST) {
      f.v[p] = ld4(src + x * ld + k);
    } else if (MODE == LOAD_XCLAMP) {
      f.v[p] = ld4g(src + (x < X ? x : X - 1) * ld + k);
    } else if (MODE == LOAD_VCLAMP) {
      // ld = K is a multiple of 4 here and so are k and Kend - Kbegin: a vector is inside or outside as a whole
      const bool in = x < X && k < Kend;
      const float4 t = ld4g(src + (x < X ? x : X - 1) * ld + (k < Kend ? k : Kend - 4));
      f.v[p] = in ? t : make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
      const bool xin = x < X;
      const float* row = src + (xin ? x : X - 1) * ld;
      float t[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const bool in = xin && k + q < Kend;
        const float val = row[k + q < Kend ? k + q : Kend - 1];
        t[q] = in ? val : 0.0f;
      }
      f.v[p] = make_float4(t[0], t[1], t[2], t[3]);
    }
  }
}
template <int BK, int XT, int NT = 256>
__device__ __forceinline__ void store_kc(const Frag<BK, XT, NT>& f, float* lds) {
  constexpr int VPR = BK / 4, RPP = NT / VPR;
  const int kq = threadIdx.x % VPR, xr = threadIdx.x / VPR;
#pragma unroll
  for (int p = 0; p < Cfg<BK, XT, NT>::NV; ++p) st4(lds + (xr + RPP * p) * Cfg<BK, XT>::KC_PITCH + 4 * kq, f.v[p]);
}

// x-contiguous source: element (x, k) at src[k*ld + x]; tile BK x XT.  LOAD_VCLAMP relies on
// X % 4 == 0 (implied by ld % 4 == 0, ld being X here): a float4 is inside or outside as a whole.
template <int BK, int XT, int MODE, int NT = 256>
__device__ __forceinline__ void load_xc(Frag<BK, XT, NT>& f, const float* __restrict__ src, size_t ld, size_t X, size_t Kend,
                                        size_t x0, size_t k0) {
  constexpr int XQ = XT / 4, KR = NT / XQ;  // float4 per k-row (32 or 16), k-rows per pass (8 or 16)
  const int xq = threadIdx.x % XQ, kr = threadIdx.x / XQ;
#pragma unroll
  for (int p = 0; p < Cfg<BK, XT, NT>::NV; ++p) {
    const size_t k = k0 + kr + KR * p, x = x0 + 4 * xq;
    if (MODE == LOAD_FAST) {
      f.v[p] = ld4(src + k * ld + x);
    } else if (MODE == LOAD_XCLAMP) {
      f.v[p] = ld4g(src + k * ld + (x < X ? x : X - 4));  // X > 32 on this path
    } else if (MODE == LOAD_VCLAMP) {
      const bool in = x < X && k < Kend;
      const float4 t = ld4g(src + (k < Kend ? k : Kend - 1) * ld + (x < X ? x : X - 4));
      f.v[p] = in ? t : make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
      const bool kin = k < Kend;
      const float* row = src + (kin ? k : Kend - 1) * ld;
      float t[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const bool in = kin && x + q < X;
        const float val = row[x + q < X ? x + q : X - 1];
        t[q] = in ? val : 0.0f;
      }
      f.v[p] = make_float4(t[0], t[1], t[2], t[3]);
    }
  }
}
template <int BK, int XT, int NT = 256>
__device__ __forceinline__ void store_xc(const Frag<BK, XT, NT>& f, float* lds) {
  constexpr int XQ = XT / 4, KR = NT / XQ;
  const int xq = threadIdx.x % XQ, kr = threadIdx.x / XQ;
  static_assert(KR % 8 == 0, "bit 2 of a thread's rows kr + KR*p is that of kr: one swizzle per thread");
  float* at = lds + kr * Cfg<BK, XT>::XC_PITCH + ((4 * xq) ^ xc_swizzle(kr));
#pragma unroll
  for (int p = 0; p < Cfg<BK, XT, NT>::NV; ++p) st4(at + KR * p * Cfg<BK, XT>::XC_PITCH, f.v[p]);
}

// LOAD_FAST and LOAD_XCLAMP as scalar base + 32-bit vector offset.  tile_offsets: the byte offset of
// each of this thread's float4 from the tile's first element at a k tile's first k, for a
// k-contiguous (KC) or an x-contiguous source - the same thread -> element map as load_kc / load_xc,
// which store_kc / store_xc rely on.  CLAMP (LOAD_XCLAMP): a row or a vector of columns that starts
// outside the operand is fetched from inside it instead (the last row; the tile's first columns) -
// its values only reach rows and columns of C that are never stored.  The offsets fit 32 bits for
// leading dimensions below 2^22, which is checked where these modes are chosen.  load_panel: the NV
// loads of a stage from the panel that starts at `panel`, a wave-uniform address:
// `global_load_dwordx4 v, v_offset, s[base]`.
template <int BK, int XT, int NT, bool KC, bool CLAMP>
__device__ __forceinline__ void tile_offsets(unsigned* off, size_t ld, size_t x0, size_t X) {
  if (KC) {
    constexpr int VPR = BK / 4, RPP = NT / VPR;
    const int kq = threadIdx.x % VPR, xr = threadIdx.x / VPR;
#pragma unroll
    for (int p = 0; p < Cfg<BK, XT, NT>::NV; ++p) {
      size_t xi = xr + RPP * p;
      if (CLAMP && x0 + xi >= X) xi = X - 1 - x0;
      off[p] = (unsigned)((xi * ld + 4 * kq) * sizeof(float));
    }
  } else {
    constexpr int XQ = XT / 4, KR = NT / XQ;
    const int xq = threadIdx.x % XQ, kr = threadIdx.x / XQ;
    const size_t xi = (CLAMP && x0 + 4 * xq >= X) ? 0 : 4 * xq;
#pragma unroll
    for (int p = 0; p < Cfg<BK, XT, NT>::NV; ++p) off[p] = (unsigned)(((size_t)(kr + KR * p) * ld + xi) * sizeof(float));
  }
}
template <int BK, int XT, int NT, bool ALIGNED>
__device__ __forceinline__ void load_panel(Frag<BK, XT, NT>& f, const float* panel, unsigned* off) {
  const char* base = reinterpret_cast<const char*>(panel);
#pragma unroll
  for (int p = 0; p < Cfg<BK, XT, NT>::NV; ++p) {
    // the empty asm keeps the 32 -> 64 bit extension of the offset next to the load: hoisted out of
    // the loop it leaves a 64-bit vector add per load behind, kept here the pair folds into the
    // load's scalar-base addressing mode
    asm volatile("" : "+v"(off[p]));
    const float* at = reinterpret_cast<const float*>(base + (size_t)off[p]);
    f.v[p] = ALIGNED ? ld4(at) : ld4g(at);
  }
}

// MFMA fragments of one 8-wide k group for the NI 32-row blocks of this wave's rows (or columns).
// KC = true: lds is [x][k]; false: [k][x] (swizzled, see Cfg).  w = the wave's coordinate along this
// side of the WG-wide wave grid.
template <bool KC, int BK, int XT, int NI, int WG>
__device__ __forceinline__ void read_frag(float (&out)[NI][4], const float* lds, int w, int kk8, int r, int h) {
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    if (KC) {
      float4 t = ld4(lds + (block_of<WG>(w, i) + r) * Cfg<BK, XT>::KC_PITCH + kk8 * 8 + 4 * h);
      out[i][0] = t.x; out[i][1] = t.y; out[i][2] = t.z; out[i][3] = t.w;
    } else {
      // bit 2 of k = 8*kk8 + 4*h + t is h: one swizzle for the lane, folded into its base address
      const float* lane_base = lds + 4 * h * Cfg<BK, XT>::XC_PITCH + ((block_of<WG>(w, 0) ^ (h << 5)) + r);
#pragma unroll
      for (int t = 0; t < 4; ++t) out[i][t] = lane_base[(kk8 * 8 + t) * Cfg<BK, XT>::XC_PITCH + 32 * WG * i];
    }
  }
}

// Linear workgroup id -> tile.  The hardware deals consecutive workgroup ids round-robin to the 8
// XCDs, each with an L2 of its own and room for 64 workgroups of the 128 x 128 tile.
// Grids that are whole 8 x 8 blocks of tiles, a multiple of eight of them (4096^3, 8192^3, the
// 2048-wide layers at batch 8192): XCD x works through blocks x, x + 8, ..., one block at a time, so
// the 64 tiles it holds share 8 panels of A and 8 of B.  FETCH_SIZE per 4096^3 launch of the eight-wave
// kernel: 765 MiB, against 2.1 GiB for the walk below (there an XCD holds two tile rows of 32 tiles
// each, which share a B panel only while the two rows stay within a few k tiles of each other, and
// on eight waves they do not); 4096^3 140.3 -> 143.6 TFLOP/s, 8192^3 138.8 -> 141.1, 2048 x 8192 x 4096
// 140.3 -> 143.7 on a box whose memory side is on the slow end of the pool.  (On the four-wave kernel of
// an earlier build the same remap was no faster for A*B and At*B and 25 % slower for A*Bt.)
// Any other grid: tiles are walked in groups of 8 tile rows, row index fastest, so that every XCD
// keeps working along ONE tile row of the group: its A panel stays put in that L2 while the B
// panels stream through.
__device__ __forceinline__ void tile_of_block(unsigned bid, unsigned tiles_m, unsigned tiles_n, unsigned& tm,
                                              unsigned& tn) {
  if (tiles_m % 8 == 0 && tiles_n % 8 == 0 && ((tiles_m / 8) * (tiles_n / 8)) % 8 == 0) {
    const unsigned x = bid & 7, q = bid >> 3;
    const unsigned blk = (q >> 6) * 8 + x, t = q & 63;
    const unsigned bm = blk % (tiles_m / 8), bn = blk / (tiles_m / 8);
    tm = bm * 8 + (t & 7);
    tn = bn * 8 + (t >> 3);
    return;
  }
  constexpr unsigned GROUP_M = 8;
  const unsigned in_group = GROUP_M * tiles_n;
  const unsigned group = bid / in_group;
  const unsigned first_m = group * GROUP_M;
  const unsigned gsize = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
  const unsigned local = bid % in_group;
  tm = first_m + local % gsize;
  tn = local / gsize;
}

// Where the k loop's code starts relative to a 32-byte boundary used to be worth up to 4 % of the
// kernel's speed (with vector address arithmetic in the loop); it is worth 0.5 % now, repeatably:
// measured on 4096^3 with the start 0 / 8 / 16 / 24 bytes past a boundary (TFLOP/s, launches back to
// back): A*B 141.9 / 142.5 / 142.9 / 142.4, A*Bt 143.4 / 143.6 / 143.8 / 143.5, At*B 141.4 / 142.2 /
// 142.0 / 141.6; the eight-wave tile at 2048^3 within 0.5 % everywhere; the 64 x 64 tile at 1024^3:
// 93.7 / 92.3 / 94.9 / 94.3, 94.1 / 92.7 / 94.5 / 93.2, 93.0 / 92.2 / 92.9 / 93.5.  Left to chance the
// start moves whenever code earlier in the file changes, so it stays pinned, per form, for the
// loops that large products spend their time in.  The best offset is a property of the loop's
// code: after a change to the loop or to what precedes it in gemm_tiles, measure the four offsets
// again.  P = offset in units of 8 bytes.
template <int P>
__device__ __forceinline__ void pin_loop_start() {
  static_assert(P >= 0 && P < 4, "offset is 0, 8, 16 or 24 bytes");
  if (P == 0) asm volatile(".p2align 5");
  if (P == 1) asm volatile(".p2align 5\n s_nop 0\n s_nop 0");
  if (P == 2) asm volatile(".p2align 5\n s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0");
  if (P == 3) asm volatile(".p2align 5\n s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0\n s_nop 0");
}
constexpr int PIN_ONLY_FAST[2][2] = {{2, 2}, {1, 2}};  // [TA][TB]; the kernel that holds no other loop
constexpr int PIN_FAST[2][2] = {{2, 2}, {1, 2}};       // the same loop in the kernel that holds all four
constexpr int PIN_XCLAMP[2][2] = {{1, 2}, {1, 1}};
constexpr int PIN_WIDE[2][2] = {{0, 0}, {0, 0}};       // the eight-wave tile (2048^3: 135.7 / 136.2 / 134.4 against 134.7 / 135.9 / 133.5 at 3)
constexpr int PIN_SMALL[2][2] = {{1, 0}, {0, 0}};      // the 64 x 64 tile (1024^3: 97.1 / 97.2 / 95.7 against 96.3 / 96.8 / 94.1 at 2)

// The k loop over tiles [kt_begin, kt_end) of one workgroup, fetching with load mode MODE.  The
// modes are separate loops on purpose: when vector and per-element loads sat behind a branch in
// ONE loop body the compiler folded them into the per-element form, which cost 19 % of the
// kernel's throughput.
// KS = 2: two sets of WGM x WGN waves share the tile and split every k tile between them, the first
// taking its k groups 0 and 1, the second 2 and 3 (the caller adds the two sets' accumulators): a
// grid that gives a CU one workgroup then puts two waves on a SIMD instead of one.
template <bool TA, bool TB, int BK, int MODE, bool ONLY_FAST, int WM, int WN, int WGM = 2, int WGN = 2, int KS = 1>
__device__ __forceinline__ void gemm_tiles(const GemmArgs& g, int kt_begin, int kt_end, size_t kbeg, size_t kend,
                                           size_t m0, size_t n0, float (*lds_a)[Cfg<BK, 32 * WM * WGM>::STAGE_FLOATS],
                                           float (*lds_b)[Cfg<BK, 32 * WN * WGN>::STAGE_FLOATS], floatx16 (&acc)[WM][WN]) {
  constexpr int TM = 32 * WM * WGM, TN = 32 * WN * WGN;  // the workgroup's tile of C
  constexpr int NT = 64 * WGM * WGN * KS;                 // its threads
  constexpr int KSTEPS = BK / 8;
  static_assert(KS == 1 || (KS == 2 && KSTEPS == 4 && !(WM == 2 && WN == 2 && WGM == 2 && WGN == 2)), "k halves: the unrolled loop only");
  // The refill (LDS stores of tile kt+1, loads of tile kt+2) sits before the LAST k-group of a k
  // tile, as one run: store A, store B, load A, load B.  Measured at 4096^3 for the refill before
  // group 0 / 1 / 2 / 3 (TFLOP/s, launches back to back): A*B 133.7 / 137.1 / 136.2 / 142.8, A*Bt
  // 135.1 / 137.3 / 137.3 / 143.8, At*B 133.0 / 135.2 / 135.0 / 141.8; the eight-wave tile at 2048^3
  // 126 / 132.5 / 133.7 / 132.6, 129 / 133.2 / 133.4 / 132.7, 125 / 126.5 / 126.5 / 131.2; the 64 x 64
  // tile does not care (1024^3: 92-95 everywhere).  Giving each operand a group of its own, or
  // spreading the refill over all four groups, measured 1-5 % below the best single position, and
  // store A, load A, store B, load B in one group 10 % below.  (While the loop still computed its
  // load addresses and LDS row bases with vector instructions the optimum was group 1 for A*B and
  // A*Bt: where the memory instructions sit matters because, issued in one run, they hold the
  // wave's MFMA issue up behind them - and so did that arithmetic.)
  constexpr int KG = KSTEPS / KS;        // k groups of a k tile that one wave multiplies
  constexpr int REFILL_AT = KG - 1;
  if (kt_begin >= kt_end) return;
  const int wave = (threadIdx.x >> 6) % (WGM * WGN), lane = threadIdx.x & 63;
  const int g0 = KS == 1 ? 0 : ((threadIdx.x >> 6) / (WGM * WGN)) * KG;  // this wave's first k group
  const int wm = wave / WGN, wn = wave % WGN;
  const int r = lane & 31, h = lane >> 5;
  // A is KC ([m][k], ld = K) unless transposed ([k][m], ld = M); B is XC ([k][n], ld = N)
  // unless transposed ([n][k], ld = K).
  const size_t lda = TA ? g.M : g.K, ldb = TB ? g.K : g.N;

  Frag<BK, TM, NT> fa;
  Frag<BK, TN, NT> fb;
  // LOAD_FAST and LOAD_XCLAMP: the address of a load is a scalar base (the tile panel at k tile kt, advanced by the
  // scalar unit) plus a per-thread 32-bit byte offset that never changes, so the loop holds no
  // vector arithmetic for its sixteen loads.  As per-thread 64-bit pointers every load cost two
  // 64-bit vector adds per k tile, and vector ALU work in this loop is paid for in matrix-core time.
  // (The buffer-descriptor form of the same idea is out: this compiler lowers the 128-bit raw buffer
  // load builtin to a 32-bit load.)
  unsigned off_a[Cfg<BK, TM, NT>::NV], off_b[Cfg<BK, TN, NT>::NV];
  const float* base_a = nullptr;
  const float* base_b = nullptr;
  constexpr bool PANEL = MODE == LOAD_FAST || MODE == LOAD_XCLAMP;
  constexpr bool ALIGNED = MODE == LOAD_FAST;
  if (PANEL) {
    tile_offsets<BK, TM, NT, !TA, MODE == LOAD_XCLAMP>(off_a, lda, m0, g.M);
    tile_offsets<BK, TN, NT, TB, MODE == LOAD_XCLAMP>(off_b, ldb, n0, g.N);
    base_a = TA ? g.A + kbeg * lda + m0 : g.A + m0 * lda + kbeg;
    base_b = TB ? g.B + n0 * ldb + kbeg : g.B + kbeg * ldb + n0;
  }
  auto load_stage = [&](int kt) {
    if (PANEL) {
      load_panel<BK, TM, NT, ALIGNED>(fa, base_a + (size_t)kt * (TA ? BK * lda : BK), off_a);
      load_panel<BK, TN, NT, ALIGNED>(fb, base_b + (size_t)kt * (TB ? BK : BK * ldb), off_b);
      return;
    }
    const size_t k0 = kbeg + (size_t)kt * BK;
    if (TA) load_xc<BK, TM, MODE, NT>(fa, g.A, lda, g.M, kend, m0, k0);
    else load_kc<BK, TM, MODE, NT>(fa, g.A, lda, g.M, kend, m0, k0);
    if (TB) load_kc<BK, TN, MODE, NT>(fb, g.B, ldb, g.N, kend, n0, k0);
    else load_xc<BK, TN, MODE, NT>(fb, g.B, ldb, g.N, kend, n0, k0);
  };
  auto store_stage = [&](int s) {
    if (TA) store_xc<BK, TM, NT>(fa, lds_a[s]); else store_kc<BK, TM, NT>(fa, lds_a[s]);
    if (TB) store_kc<BK, TN, NT>(fb, lds_b[s]); else store_xc<BK, TN, NT>(fb, lds_b[s]);
  };

  // Software pipeline over the k tiles.  While tile kt is multiplied out of LDS stage s:
  //   * the registers hold tile kt+1 (its global loads were issued one iteration ago);
  //   * before k-group REFILL_AT of tile kt those registers are stored to stage s^1 and the global
  //     loads of tile kt+2 are issued, so that both the LDS stores and the load issue hide behind
  //     the last MFMA group (16 MFMAs = 1024 cycles) instead of sitting between the MFMA block
  //     and the barrier (see REFILL_AT above for where in the block it goes);
  //   * MFMA fragments are read from LDS one k-group ahead of the MFMAs that consume them.
  // The scheduling barriers keep the compiler from sinking the reads and stores back down.
  load_stage(kt_begin);
  store_stage(0);
  if (kt_begin + 1 < kt_end) load_stage(kt_begin + 1);
  __syncthreads();

  constexpr bool BIG = WM == 2 && WN == 2 && WGM == 2 && WGN == 2;
  constexpr bool WIDE = WGM * WGN == 8;
  if (MODE == LOAD_FAST)
    pin_loop_start<WIDE ? PIN_WIDE[TA][TB] : !BIG ? PIN_SMALL[TA][TB] : ONLY_FAST ? PIN_ONLY_FAST[TA][TB] : PIN_FAST[TA][TB]>();
  if (MODE == LOAD_XCLAMP) pin_loop_start<BIG ? PIN_XCLAMP[TA][TB] : PIN_SMALL[TA][TB]>();
  // One k tile out of a stage that is a compile-time constant: the loop that uses this is unrolled
  // by two, so that every LDS address is the lane's base plus an immediate - a run-time stage has
  // its offset added to four base registers in every k tile.
  auto k_tile = [&](int kt, auto stage) {
    constexpr int s = decltype(stage)::value;
    float a[2][WM][4], b[2][WN][4];
    read_frag<!TA, BK, TM, WM, WGM>(a[0], lds_a[s], wm, g0, r, h);
    read_frag<TB, BK, TN, WN, WGN>(b[0], lds_b[s], wn, g0, r, h);
#pragma unroll
    for (int kk8 = 0; kk8 < KG; ++kk8) {
      const int cur = kk8 & 1, nxt = cur ^ 1;
      if (kk8 + 1 < KG) {
        read_frag<!TA, BK, TM, WM, WGM>(a[nxt], lds_a[s], wm, g0 + kk8 + 1, r, h);
        read_frag<TB, BK, TN, WN, WGN>(b[nxt], lds_b[s], wn, g0 + kk8 + 1, r, h);
      }
      if (kk8 == REFILL_AT) {
        // stage s^1 was last read in the previous k tile, which ended with a barrier
        if (kt + 1 < kt_end) store_stage(s ^ 1);
        if (kt + 2 < kt_end) load_stage(kt + 2);
      }
      __builtin_amdgcn_sched_barrier(0);
      // the wave that is in its MFMA block wins the issue arbitration against the wave of the other
      // workgroup on the same SIMD, which is fetching or waiting (measured: +2 % on A*B, +1 % on At*B)
      __builtin_amdgcn_s_setprio(1);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][i][t], b[cur][j][t], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();  // stage s^1 is complete, stage s is free; also leaves LDS free for whoever runs next
  };
  // Unrolled for the eight-wave and the 64 x 64 tile (2048^3 132.5 -> 135.3, 1024^3 94 -> 96.5
  // TFLOP/s); the four-wave 128 x 128 loop measured 0.7-1.3 % slower unrolled for A*B and A*Bt
  // (its second copy starts wherever it happens to fall) and keeps the run-time stage.
  if (BIG) {
    // (the same body written out: as a call of k_tile with a run-time stage this loop compiled to
    // something 5 % slower)
    for (int kt = kt_begin; kt < kt_end; ++kt) {
      const int s = (kt - kt_begin) & 1;
      float a[2][WM][4], b[2][WN][4];
      read_frag<!TA, BK, TM, WM, WGM>(a[0], lds_a[s], wm, 0, r, h);
      read_frag<TB, BK, TN, WN, WGN>(b[0], lds_b[s], wn, 0, r, h);
#pragma unroll
      for (int kk8 = 0; kk8 < KSTEPS; ++kk8) {
        const int cur = kk8 & 1, nxt = cur ^ 1;
        if (kk8 + 1 < KSTEPS) {
          read_frag<!TA, BK, TM, WM, WGM>(a[nxt], lds_a[s], wm, kk8 + 1, r, h);
          read_frag<TB, BK, TN, WN, WGN>(b[nxt], lds_b[s], wn, kk8 + 1, r, h);
        }
        if (kk8 == REFILL_AT) {
          if (kt + 1 < kt_end) store_stage(s ^ 1);
          if (kt + 2 < kt_end) load_stage(kt + 2);
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][i][t], b[cur][j][t], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
      }
      __syncthreads();
    }
  } else {
    for (int kt = kt_begin; kt < kt_end; kt += 2) {
      k_tile(kt, std::integral_constant<int, 0>());
      if (kt + 1 < kt_end) k_tile(kt + 1, std::integral_constant<int, 1>());
    }
  }
}

// k tiles [ka, kb) (counted from kbeg; the chunk ends at kend) of the tile at (m0, n0), each
// stretch with the cheapest load mode that is valid for it:
//   interior tile of float4-loadable, 16-byte aligned operands: LOAD_FAST for the complete k
//   tiles, LOAD_VCLAMP for the k remainder;
//   otherwise (edge tile, base only float-aligned, rows of odd length): LOAD_XCLAMP for the k
//   tiles that end before the operand's last k index, then LOAD_VCLAMP or, for rows of odd length,
//   LOAD_SCALAR for the rest (one tile, or the k remainder).
// ONLY_FAST: the host has checked that every k tile of every tile qualifies for LOAD_FAST (M and N
// multiples of 128, every k chunk a multiple of BK, operands float4-loadable and 16-byte aligned);
// the kernel then contains that one loop and nothing else.
template <bool TA, bool TB, int BK, bool ONLY_FAST, int WM, int WN, int WGM = 2, int WGN = 2, int KS = 1>
__device__ __forceinline__ void gemm_k_range(const GemmArgs& g, int ka, int kb, size_t kbeg, size_t kend, size_t m0,
                                             size_t n0, float (*lds_a)[Cfg<BK, 32 * WM * WGM>::STAGE_FLOATS],
                                             float (*lds_b)[Cfg<BK, 32 * WN * WGN>::STAGE_FLOATS], floatx16 (&acc)[WM][WN]) {
  if (ONLY_FAST) {
    gemm_tiles<TA, TB, BK, LOAD_FAST, true, WM, WN, WGM, WGN, KS>(g, ka, kb, kbeg, kend, m0, n0, lds_a, lds_b, acc);
    return;
  }
  const bool vec = g.a_vec && g.b_vec;
  const bool fast = vec && m0 + 32 * WM * WGM <= g.m_fast && n0 + 32 * WN * WGN <= g.N;
  const int kfull = (int)((kend - kbeg) / BK);             // complete k tiles of the chunk
  const int before_last = (int)((g.K - 1 - kbeg) / BK);    // k tiles that end before index K - 1
  int e1 = fast ? (kb < kfull ? kb : kfull) : ka;
  if (e1 < ka) e1 = ka;
  int e2 = e1;
  // (the x-clamped loop addresses a tile panel with 32-bit byte offsets, like the fast one)
  const bool narrow_ld = (TA ? g.M : g.K) < (size_t(1) << 22) && (TB ? g.K : g.N) < (size_t(1) << 22);
  if (!fast && narrow_ld) {
    e2 = kb < before_last ? kb : before_last;
    if (e2 < e1) e2 = e1;
  }
  const int e3 = vec ? kb : e2;
  gemm_tiles<TA, TB, BK, LOAD_FAST, false, WM, WN, WGM, WGN, KS>(g, ka, e1, kbeg, kend, m0, n0, lds_a, lds_b, acc);
  gemm_tiles<TA, TB, BK, LOAD_XCLAMP, false, WM, WN, WGM, WGN, KS>(g, e1, e2, kbeg, kend, m0, n0, lds_a, lds_b, acc);
  gemm_tiles<TA, TB, BK, LOAD_VCLAMP, false, WM, WN, WGM, WGN, KS>(g, e2, e3, kbeg, kend, m0, n0, lds_a, lds_b, acc);
  gemm_tiles<TA, TB, BK, LOAD_SCALAR, false, WM, WN, WGM, WGN, KS>(g, e3, kb, kbeg, kend, m0, n0, lds_a, lds_b, acc);
}

// A workgroup that computes one whole tile of C (or, with g.splits > 1, one k chunk of it as a raw
// partial product): blockIdx.x = tile, blockIdx.y = k chunk.
template <bool TA, bool TB, int BK, bool ONLY_FAST, int WM, int WN, int WGM = 2, int WGN = 2, int KS = 1>
__device__ __forceinline__ void gemm_whole_tile(const GemmArgs& g, float (*lds_a)[Cfg<BK, 32 * WM * WGM>::STAGE_FLOATS],
                                                float (*lds_b)[Cfg<BK, 32 * WN * WGN>::STAGE_FLOATS]) {
  constexpr int TM = 32 * WM * WGM, TN = 32 * WN * WGN;
  unsigned tm, tn;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  const size_t m0 = (size_t)tm * TM, n0 = (size_t)tn * TN;
  const size_t kbeg = (size_t)blockIdx.y * g.k_chunk;
  const size_t kend = kbeg + g.k_chunk < g.K ? kbeg + g.k_chunk : g.K;
  const int ktiles = (int)((kend - kbeg + BK - 1) / BK);

  const int wave = (threadIdx.x >> 6) % (WGM * WGN), lane = threadIdx.x & 63;
  const int wm = wave / WGN, wn = wave % WGN;
  const int r = lane & 31, h = lane >> 5;

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  gemm_k_range<TA, TB, BK, ONLY_FAST, WM, WN, WGM, WGN, KS>(g, 0, ktiles, kbeg, kend, m0, n0, lds_a, lds_b, acc);

  if (KS == 2) {
    // the second set of waves hands its accumulators over through LDS (every k loop ends with a barrier, so
    // the stages are free), one of its WM block rows at a time, and is done; the first adds them - always
    // in this order - and writes the tile
    static_assert(KS == 1 || WN * WGM * WGN * 1024 <= 2 * Cfg<BK, 32 * WM * WGM>::STAGE_FLOATS, "a block row of accumulators fits stage memory");
    float* red = &lds_a[0][0];
    const bool second = (threadIdx.x >> 6) >= WGM * WGN;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      if (second) {
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) red[((wave * WN + j) * 16 + v) * 64 + lane] = acc[i][j][v];
      }
      __syncthreads();
      if (!second) {
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[i][j][v] += red[((wave * WN + j) * 16 + v) * 64 + lane];
      }
      if (i + 1 < WM) __syncthreads();
    }
    if (second) return;
  }

  // Epilogue.  Accumulator register v of lane (r, h) in block (i, j) is
  //   row = 8*(v/4) + 4*h + v%4,  col = r   within the 32 x 32 block at (block_of(wm, i), block_of(wn, j)).
  // No load may sit between two stores: C, pre_act and dst can be the same memory as far as the
  // compiler knows, so a `beta * C[idx]` read after a store waits for that store, 64 times in a
  // row (measured: 7.5 us per workgroup, more than a 128x128x128 product itself).  Hence: first
  // every read (C for beta), then only stores; and the common plain case is its own loop.
  const bool raw = g.splits > 1;
  float* dst = raw ? g.partial + (size_t)blockIdx.y * g.M * g.N : g.C;
  const bool interior = m0 + TM <= g.M && n0 + TN <= g.N;
  auto for_each = [&](auto&& fn) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const size_t col = n0 + block_of<WGN>(wn, j) + r;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const size_t row = m0 + block_of<WGM>(wm, i) + 8 * (v / 4) + 4 * h + (v % 4);
          if (interior || (row < g.M && col < g.N)) fn(i, j, v, row * g.N + col, col);
        }
      }
  };
  if (raw || (g.beta == 0.0f && !g.bias && !g.pre_act && !g.relu && !g.mask)) {
    for_each([&](int i, int j, int v, size_t idx, size_t) { dst[idx] = acc[i][j][v]; });
    return;
  }
  // A tile inside the matrix with nothing to read back but the bias (a Linear forward with its ReLU): one
  // wave-uniform row pointer per accumulator register and one 32-bit lane offset for all of them
  // (8192 x 2048 x 2048 with bias and ReLU, launches back to back: 499 -> 486 us, the plain product's time).
  if (interior && g.beta == 0.0f && !g.mask && g.N < (size_t(1) << 28)) {
    const int uw = __builtin_amdgcn_readfirstlane(wave);
    const int uwm = uw / WGN, uwn = uw % WGN;
    const unsigned lane_off = (unsigned)(4 * h) * (unsigned)g.N + (unsigned)r;
    const bool relu = g.relu != 0;
    float bv[WN];
#pragma unroll
    for (int j = 0; j < WN; ++j) bv[j] = g.bias ? g.bias[n0 + block_of<WGN>(wn, j) + r] : 0.0f;
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const size_t first = (m0 + block_of<WGM>(uwm, i)) * g.N + n0 + block_of<WGN>(uwn, j);  // wave-uniform
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const size_t at = first + (size_t)(8 * (v / 4) + v % 4) * g.N;
          float val = acc[i][j][v];
          if (g.bias) val = val + bv[j];
          if (g.pre_act) (g.pre_act + at)[lane_off] = val;
          const float rl = (val >= 0.0f ? 1.0f : 0.0f) * val;
          (dst + at)[lane_off] = relu ? rl : val;
        }
      }
    return;
  }
  if (g.mask)
    for_each([&](int i, int j, int v, size_t idx, size_t) {
      acc[i][j][v] = (g.mask[idx] >= 0.0f ? 1.0f : 0.0f) * acc[i][j][v];
    });
  if (g.beta != 0.0f)
    for_each([&](int i, int j, int v, size_t idx, size_t) { acc[i][j][v] = g.beta * g.C[idx] + acc[i][j][v]; });
  if (g.bias) {
    float bv[WN];
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const size_t col = n0 + block_of<WGN>(wn, j) + r;
      bv[j] = col < g.N ? g.bias[col] : 0.0f;
    }
    for_each([&](int i, int j, int v, size_t, size_t) { acc[i][j][v] = acc[i][j][v] + bv[j]; });
  }
  if (g.pre_act) for_each([&](int i, int j, int v, size_t idx, size_t) { g.pre_act[idx] = acc[i][j][v]; });
  if (g.relu)
    for_each([&](int i, int j, int v, size_t idx, size_t) {
      const float val = acc[i][j][v];
      dst[idx] = (val >= 0.0f ? 1.0f : 0.0f) * val;
    });
  else
    for_each([&](int i, int j, int v, size_t idx, size_t) { dst[idx] = acc[i][j][v]; });
}

// Launches the spread-tail kernel and its fix-up (gemm_spread.hip).
// gemm_skinny.hip: K <= 12, or A^T * B with N <= 16.  Returns 0 (not taken), 1 (done, *rc holds the
// result) or 2 (partials of g.splits k ranges are in the workspace: the caller combines them).
int gemm_skinny_launch(slhip_ctx* ctx, bool ta, bool tb, GemmArgs& g, int32_t* rc);
// The tall-A, at most 32 columns kernel (gemm_tall.hip), same convention.
int gemm_tall_launch(slhip_ctx* ctx, bool ta, bool tb, GemmArgs& g, int32_t* rc);
// The K <= 12 kernel alone, with the mask of the product given as bits (row-major, 32 columns to a
// word) or NULL.  Returns 1 if it took the product (*rc = launch status), else 0.
int gemm_short_k_launch(slhip_ctx* ctx, bool ta, bool tb, const GemmArgs& g, const uint32_t* bits, int32_t* rc);

// gemm_wide.hip: the 128 x 128 tile on eight waves, g planned as for the four-wave kernel.
int32_t gemm_wide_launch(slhip_ctx* ctx, bool ta, bool tb, bool only_fast, const GemmArgs& g);
// gemm_wide.hip: the 64 x 64 tile on eight waves, two sets of four that split every k tile; g planned for 64 x 64 tiles, no k split.
int32_t gemm_small8_launch(slhip_ctx* ctx, bool ta, bool tb, bool only_fast, const GemmArgs& g);
// gemm_wide.hip: the 128 x 128 tile on sixteen waves, two sets of eight that split every k tile; g planned for 128 x 128 tiles, no k split.
int32_t gemm_wide16_launch(slhip_ctx* ctx, bool ta, bool tb, bool only_fast, const GemmArgs& g);

int32_t gemm_spread_launch(slhip_ctx* ctx, bool ta, bool tb, bool only_fast, bool small_tile, const GemmArgs& g,
                           const SpreadArgs& sp, size_t workers, size_t tail_tiles, bool wide);

}  // namespace slhip
