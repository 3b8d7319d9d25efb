// Tiles, loaders and kernels of the FP32 GEMM (gemm.hip describes them) for the two files that instantiate them: gemm.hip
// (FP32 MFMA) and gemm_split.hip (the same products through bf16 pieces).
#pragma once
#include <algorithm>
#include "common.h"

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// K depth of one LDS stage (BKT, 16 or 32) is a template parameter; a k-contiguous operand tile has
// row stride BKT+4 words (20 or 36: both = 4 mod 32, see above).

struct GemmArgs {
  const float *A, *B;
  float *C;
  int M, N, K;
  int lda, ldb, ldc;
  int acc;
  int kchunk;              // K range per blockIdx.z when splitting (multiple of BK), else K
  int splits;              // >1: write partials to P[z][M][N]
  float *Pp;
  int64_t sA, sB, sC;      // batch strides (elements); batch index = blockIdx.z when splits == 1
  int nbm, nbn;
  // optional second K segment: C = A.B (+) A2.B2 with the same M, N and operand orientation (K2 = 0: none)
  const float *A2, *B2;
  int K2, lda2, ldb2;
  // banded batch (gemm_direct<..., BAND>): batch member z = zb * zdiv + zh takes A + z*sA, B + zb*sB + (zh/zgroup)*sB2 and
  // C + zb*sC + zh*sC2, and the row tile at m0 contracts over k in [band start of m0, m0 + BM) only: the product of a
  // causal (optionally windowed) score-gradient matrix with the key rows, one (sequence, head) per batch member
  int zdiv, zgroup, window;
  int64_t sB2, sC2;
  // further whole K segments (gemm_direct<..., MSEG>): C = A.B + xA[0].xB[0] (+ xA[1].xB[1]), every K a multiple of the
  // K step, same M, N and operand orientation: the dX of sibling projections of one input as one product
  const float *xA[2], *xB[2];
  int xK[2], xlda[2], xldb[2], nx;
  // C = D + A.B: the matrix the product is added to when it is not C's own old contents (layout of C, batch stride sD;
  // null: none). With K splits the reduce kernel adds it. scaled: C = dscale * D + pscale * A.B (the Newton-Schulz
  // combines b A + c A.A and a X + B.X in the products' own write-back).
  const float *D;
  int64_t sD;
  int scaled;
  float dscale, pscale;
  // banded batch only: the (cos, sin) table ([M][N/2] pairs) of the rotation the rows of the other operand's source went
  // through; the write-back then applies that rotation's backward to each row of C (pairs (j, j + N/2)). Null: none.
  const float *rope;
  // banded batch with splits > 1 (small launches): blockIdx.y cuts every row tile's K range into `splits` parts, each written
  // unrotated and unaccumulated to Pp + blockIdx.y * sP (laid out as C); band_dq_reduce adds them up, rotates and accumulates
  int64_t sP;
};

// Which output tile (pm, pn) and which K split or batch member (z) a workgroup works on. Workgroups are handed
// to the 8 XCDs round-robin in dispatch order (x fastest, then z), each XCD with its own L2. Renumber so that one XCD
// walks a contiguous range of tiles: neighbours then share their A row panel in that L2. With K splits the range is over
// the split-major list of (split, tile) pairs, so the workgroups resident on an XCD at one time are (nearly) all the
// tiles of ONE split, walking the same K range: every operand slab they load is shared through that L2. (With the tiles
// renumbered per split only, every XCD held a few tiles of every split in flight and dW missed L2 for 6x its operands.)
__device__ __forceinline__ void tile_of_workgroup(const GemmArgs &a, int &pm, int &pn, int &z) {
  const int nblk = a.nbm * a.nbn;
  int pid;
  if (a.splits > 1) {
    const int total = nblk * a.splits, lin = blockIdx.x + blockIdx.z * nblk;
    const int xcd = lin % 8, idx = lin / 8, base = total / 8, rem = total % 8;
    const int w = xcd * base + (xcd < rem ? xcd : rem) + idx;
    z = w / nblk;
    pid = w % nblk;
  } else {
    const int p = blockIdx.x;
    const int xcd = p % 8, idx = p / 8, base = nblk / 8, rem = nblk % 8;
    pid = xcd * base + (xcd < rem ? xcd : rem) + idx;
    z = blockIdx.z;
  }
  // Tiles are numbered in bands of 8 tile rows, M fastest inside a band: the ~64 workgroups resident on an XCD then
  // cover about 8 rows x 8 columns of tiles instead of 1 x 64, and each K slab of A and of B they load is shared by 8
  // of them through the L2 (a wide output such as the readout's streamed all of B once per tile row before: 14.4 GB of
  // L2 misses per launch for a 113 MB weight matrix, 4.0 GB with the bands).
  // Outputs at most 8 tiles wide keep plain N-fastest order: a row of tiles is then no more than the resident set and
  // the bands only add A panels in flight (measured: 5-20 % more L2 misses for the N = 576 products).
  if (a.nbn <= 8) { pm = pid / a.nbn; pn = pid % a.nbn; return; }
  const int band = pid / (8 * a.nbn), first = band * 8, rows = min(8, a.nbm - first), in_band = pid - band * 8 * a.nbn;
  pm = first + in_band % rows;
  pn = in_band / rows;
}

// One operand tile of R rows x BKT k, kept in LDS as [row][BKT+4] with the 16-byte K chunks of a row XOR-swizzled by
// (row/8) mod (BKT/4). KC: k contiguous in memory (element (r,k) at p[r*ld + k]), copied with one ds_write_b128 per
// float4. Otherwise row contiguous (element (r,k) at p[k*ld + r]): eight lanes read one 128-byte line of a k-row and
// each float4 is transposed into LDS with four scalar stores; the swizzle makes those stores hit 32 distinct banks per
// half-wavefront (measured: 2 cycles per 64-lane store, no conflicts). Either way the MFMA inputs of four consecutive
// steps come from one ds_read_b128. Measured with the LDS bank-conflict counters: gfx950 serves a b128 read 16 lanes
// per cycle over 64 banks, and this swizzle makes the fetch take 12 cycles instead of the 4 of an unswizzled
// [row][BKT+4] tile. A conflict-free variant (k-major tiles for row-contiguous operands, unswizzled copies) was built
// and changed no kernel time: the LDS pipe is far from saturated (about 15 % busy), so the layout stays.
template <int R, bool KC, bool VEC, int NT, int BKT>
struct Tile {
  static constexpr int KS = BKT + 4;
  static constexpr int KQ = BKT / 4;           // float4 chunks along K
  static constexpr int UNITS = R * KQ;         // float4 units per tile
  static constexpr int PER = (UNITS + NT - 1) / NT;   // per thread (the last round may be partial)
  static constexpr bool FULL = (UNITS % NT == 0);
  static constexpr int LDS_WORDS = R * KS;
  static_assert(R % 32 == 0, "tile rows must be a multiple of 32");

  // unit u of a row-contiguous tile: float4 column c4 (rows 4*c4..4*c4+3) at k-row kk
  __device__ static __forceinline__ void rc_unit(int u, int &c4, int &kk) {
    c4 = (u / (8 * BKT)) * 8 + (u & 7);
    kk = (u >> 3) % BKT;
  }

  // registers <- global, zero outside [0,Rtot) x [k0,kend)
  __device__ static __forceinline__ void load(v4f (&reg)[PER], const float *__restrict__ p, int ld, int r0, int Rtot,
                                              int k0, int kend, int tid) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int u = tid + i * NT;
      v4f v = {0.f, 0.f, 0.f, 0.f};
      if (!FULL && u >= UNITS) { reg[i] = v; continue; }
      if (KC) {
        int r = r0 + u / KQ, k = k0 + (u % KQ) * 4;
        if (r < Rtot) {
          const float *q = p + (size_t)r * ld + k;
          if (VEC) { if (k < kend) v = *reinterpret_cast<const v4f *>(q); }
          else {
#pragma unroll
            for (int j = 0; j < 4; j++) if (k + j < kend) v[j] = q[j];
          }
        }
      } else {
        int c4, kk;
        rc_unit(u, c4, kk);
        int k = k0 + kk, r = r0 + c4 * 4;
        if (k < kend) {
          const float *q = p + (size_t)k * ld + r;
          if (VEC) { if (r < Rtot) v = *reinterpret_cast<const v4f *>(q); }
          else {
#pragma unroll
            for (int j = 0; j < 4; j++) if (r + j < Rtot) v[j] = q[j];
          }
        }
      }
      reg[i] = v;
    }
  }
  __device__ static __forceinline__ void store(const v4f (&reg)[PER], float *lds, int tid) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int u = tid + i * NT;
      if (!FULL && u >= UNITS) continue;
      if (KC) {
        int row = u / KQ, chunk = u % KQ;
        *reinterpret_cast<v4f *>(lds + row * KS + 4 * (chunk ^ ((row >> 3) & (KQ - 1)))) = reg[i];
      } else {
        int c4, kk;
        rc_unit(u, c4, kk);
#pragma unroll
        for (int j = 0; j < 4; j++) {
          int row = c4 * 4 + j;
          lds[row * KS + 4 * ((kk >> 2) ^ ((row >> 3) & (KQ - 1))) + (kk & 3)] = reg[i][j];
        }
      }
    }
  }
  // MFMA inputs of this lane for the four steps of K-run c (0 .. BKT/8-1): row = tile row, g = lane/32
  __device__ static __forceinline__ v4f fetch(const float *lds, int row, int c, int g) {
    return *reinterpret_cast<const v4f *>(lds + row * KS + 4 * ((2 * c + g) ^ ((row >> 3) & (KQ - 1))));
  }
};

template <int BM, int BN, int WM, int WN, int BKT, int KIND, bool VEC, bool SEG2 = false>
__global__ __launch_bounds__(WM *WN * 64) void gemm_kernel(GemmArgs a) {
  constexpr int BK = BKT;
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tile must be whole MFMA tiles");
  constexpr bool AKC = (KIND != GT_TN), BKC = (KIND == GT_NT);
  using TA = Tile<BM, AKC, VEC, NT, BKT>;
  using TB = Tile<BN, BKC, VEC, NT, BKT>;
  __shared__ __attribute__((aligned(16))) float sA[TA::LDS_WORDS];
  __shared__ __attribute__((aligned(16))) float sB[TB::LDS_WORDS];

  int pm, pn, z;
  tile_of_workgroup(a, pm, pn, z);
  const int m0 = pm * BM, n0 = pn * BN;
  const float *A = a.A, *B = a.B;
  int k0 = 0, kend = a.K;
  if (a.splits > 1) { k0 = z * a.kchunk; kend = min(a.K, k0 + a.kchunk); }
  else { A += z * a.sA; B += z * a.sB; }

  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / WN, wn = wave % WN;
  const int g = lane / 32, l32 = lane % 32;

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  v4f ra[TA::PER], rb[TB::PER];
  TA::load(ra, A, a.lda, m0, a.M, k0, kend, tid);
  TB::load(rb, B, a.ldb, n0, a.N, k0, kend, tid);

  // MFMAs of one K step over the tiles in LDS
#define GEMM_MFMA_STEP()                                                                                          \
  _Pragma("unroll") for (int c = 0; c < BKT / 8; c++) {                                                           \
    v4f fa[TM], fb[TN];                                                                                           \
    _Pragma("unroll") for (int i = 0; i < TM; i++) fa[i] = TA::fetch(sA, wm * (TM * 32) + i * 32 + l32, c, g);     \
    _Pragma("unroll") for (int j = 0; j < TN; j++) fb[j] = TB::fetch(sB, wn * (TN * 32) + j * 32 + l32, c, g);     \
    _Pragma("unroll") for (int s = 0; s < 4; s++)                                                                 \
      _Pragma("unroll") for (int i = 0; i < TM; i++)                                                              \
        _Pragma("unroll") for (int j = 0; j < TN; j++)                                                            \
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);               \
  }
  if (!SEG2) {
    for (int k = k0; k < kend; k += BK) {
      __syncthreads();                     // previous step's LDS reads are done
      TA::store(ra, sA, tid);
      TB::store(rb, sB, tid);
      __syncthreads();
      if (k + BK < kend) {
        TA::load(ra, A, a.lda, m0, a.M, k + BK, kend, tid);
        TB::load(rb, B, a.ldb, n0, a.N, k + BK, kend, tid);
      }
      GEMM_MFMA_STEP()
    }
  } else {
    // The K loop runs over two segments (operand pointers, leading dimensions, K range); the step after the last one
    // of the first segment is the first one of the second, so the pipeline of loads never drains in between.
    int lda = a.lda, ldb = a.ldb, k = k0;
    bool second = false;
    for (;;) {
      __syncthreads();
      TA::store(ra, sA, tid);
      TB::store(rb, sB, tid);
      __syncthreads();
      k += BK;
      bool more = k < kend;
      if (!more && !second) {
        second = more = true;
        A = a.A2; B = a.B2; lda = a.lda2; ldb = a.ldb2; k = 0; kend = a.K2;
      }
      if (more) {
        TA::load(ra, A, lda, m0, a.M, k, kend, tid);
        TB::load(rb, B, ldb, n0, a.N, k, kend, tid);
      }
      GEMM_MFMA_STEP()
      if (!more) break;
    }
  }
#undef GEMM_MFMA_STEP

  // accumulator register r of lane (g,l32) is C[8*(r/4) + 4*g + r%4][l32] of its 32x32 tile
  float *C;
  int ldc;
  bool add;
  if (a.splits > 1) { C = a.Pp + (size_t)z * a.M * a.N; ldc = a.N; add = false; }
  else { C = a.C + z * a.sC; ldc = a.ldc; add = a.acc != 0 || a.D != nullptr; }
  const float *Cold = (a.D && a.splits == 1) ? a.D + z * a.sD : C;
  const bool scaled = a.scaled && a.splits == 1;
  // When accumulating, the sixteen old values of a 32x32 tile are loaded together (from clamped, always valid
  // addresses) before the first store: a load placed after a store to the same array waits for it, and one round trip
  // per element is what an interleaved read-add-write loop would pay.
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int col = n0 + wn * (TN * 32) + j * 32 + l32;
      const int rbase = m0 + wm * (TM * 32) + i * 32 + 4 * g;
      float old[16];
      if (add) {
        const float *cc = Cold + min(col, a.N - 1);
#pragma unroll
        for (int r = 0; r < 16; r++) old[r] = cc[(size_t)min(rbase + 8 * (r / 4) + (r % 4), a.M - 1) * ldc];
      }
      if (col >= a.N) continue;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int row = rbase + 8 * (r / 4) + (r % 4);
        if (row < a.M) C[(size_t)row * ldc + col] = !add ? acc[i][j][r] : scaled ? a.dscale * old[r] + a.pscale * acc[i][j][r] : old[r] + acc[i][j][r];
      }
    }
}

// The same contraction with both operand tiles brought from global memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, no ds_write), double-buffered, one barrier per K step of 32.
// A wave-level load writes 64 x 16 bytes contiguously, so tiles are unpadded. A k-contiguous operand is kept as
// [row][8 chunks] with the swizzle (chunk ^ row%8) applied by choosing which global chunk each lane fetches, and
// read back with one ds_read_b128 per four MFMA steps; a row-contiguous operand is kept as it lies in memory,
// [k][R], and read with four ds_read_b32 (consecutive lanes, consecutive words). K (and every split of it) must be a
// multiple of 32 and M, N multiples of 4 where they are the contiguous index; rows or columns past the edge are read
// from the last valid ones (they only reach parts of C that are not stored).
__device__ __forceinline__ void load_to_lds16(const float *src, float *wave_base) {
  // 16 bytes per lane to wave_base + lane*16 (wave_base is wave-uniform). The host pass of the compiler does not know
  // the builtin, so it only exists in the device pass.
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void *)wave_base, 16, 0, 0);
#endif
}

template <int R, bool KC, int NT, int BKD>
struct DirectTile {
  static constexpr int CPR = BKD / 4;              // 16-byte chunks per row of a k-contiguous tile (8 or 4)
  static constexpr int CH = R * CPR;               // chunks per stage (R rows x BKD k)
  static constexpr int WL = CH / 64;               // wave-level loads per stage, dealt round-robin to the wavefronts
  static constexpr int NW = NT / 64;
  static constexpr int PER = (WL + NW - 1) / NW;   // per wavefront; when WL is not a multiple of NW the spare slots
  static_assert(CH % 64 == 0, "tile must be a whole number of wave loads");   // repeat an earlier load (same data, same place)
  __device__ static __forceinline__ int load_index(int wave, int i) { return (wave + i * NW) % WL; }
  // XOR swizzle of a row's chunks: any 16 consecutive rows put a given chunk on 16 different bank groups
  __device__ static __forceinline__ int sw(int row) { return CPR == 8 ? (row & 7) : ((row & 3) ^ ((row >> 2) & 3)); }
  // Source of this lane's chunk in load i of its wavefront, for the stage that starts at k = 0, as a wave-uniform origin
  // (the tile's first row or column) plus this lane's byte offset from it, which fits 32 bits and never changes: a
  // stage's loads are then "scalar base + lane offset" and moving on by a stage is scalar arithmetic.
  __device__ static __forceinline__ const float *origin(const float *p, int ld, int r0) { return KC ? p + (size_t)r0 * ld : p + r0; }
  __device__ static __forceinline__ unsigned off(int ld, int r0, int Rtot, int wave, int i, int lane) {
    const int slot = load_index(wave, i) * 64 + lane;
    if (KC) {
      const int row = slot / CPR, c = (slot % CPR) ^ sw(row);
      return (unsigned)(((size_t)(min(r0 + row, Rtot - 1) - r0) * ld + 4 * c) * sizeof(float));
    }
    const int k = slot / (R / 4), c4 = slot % (R / 4);
    return (unsigned)(((size_t)k * ld + (min(r0 + 4 * c4, Rtot - 4) - r0)) * sizeof(float));
  }
  __device__ static __forceinline__ const float *src(const float *p, int ld, int r0, int Rtot, int wave, int i, int lane) {
    return reinterpret_cast<const float *>(reinterpret_cast<const char *>(origin(p, ld, r0)) + off(ld, r0, Rtot, wave, i, lane));
  }
  // The same for a second K segment of K2 <= BKD (a multiple of 8) that fills one stage partly: chunks past K2 repeat
  // valid ones (they are loaded but never fed to an MFMA), so nothing is read outside the operand.
  __device__ static __forceinline__ const float *src2(const float *p, int ld, int r0, int Rtot, int K2, int wave, int i, int lane) {
    const int slot = load_index(wave, i) * 64 + lane;
    if (KC) {
      const int row = slot / CPR, c = ((slot % CPR) ^ sw(row)) % (K2 / 4);
      return p + (size_t)min(r0 + row, Rtot - 1) * ld + 4 * c;
    }
    const int k = (slot / (R / 4)) % K2, c4 = slot % (R / 4);
    return p + (size_t)k * ld + min(r0 + 4 * c4, Rtot - 4);
  }
  __device__ static __forceinline__ size_t stage_step(int ld) { return KC ? (size_t)BKD : (size_t)BKD * ld; }
  // MFMA inputs of this lane for the four steps of K-run c: tile row `row`, g = lane/32 (k = 8c + 4g + s at step s)
  __device__ static __forceinline__ v4f fetch(const float *lds, int row, int c, int g) {
    if (KC) return *reinterpret_cast<const v4f *>(lds + row * BKD + 4 * ((2 * c + g) ^ sw(row)));
    const float *q = lds + (8 * c + 4 * g) * R + row;
    return v4f{q[0], q[R], q[2 * R], q[3 * R]};
  }
};


// ---- FP32 products from bf16 pieces ---------------------------------------------------------------------------------
// An FP32 number is the exact sum of three bf16 numbers (8 significant bits each: h = x cut to its upper 16 bits,
// m = x - h cut likewise, l = x - h - m, which has at most 8 significant bits left). A product of two FP32 numbers
// is then nine bf16 products, each exact in FP32; the three smallest (m.l, l.m, l.l: below 2^-24 of the whole) are
// left out, as an FP32 multiply-add rounds away as much. v_mfma_f32_32x32x16_bf16 does 16 times the multiply-adds per cycle of
// v_mfma_f32_32x32x2_f32, so the six products per pair cost 3/8 of the FP32 instruction's time, and against float64 the
// result is as close as the FP32 MFMA's (the accumulation is FP32 either way). Infinities and NaNs come out as NaN
// (inf - inf in the split).
#include "bf16_pieces.h"

// The MFMA inputs of one lane from an operand tile as DirectTile leaves it in LDS (FP32): the 8 consecutive k
// (16c + 8g ...) of `row`, cut into pieces here, in registers, by every wavefront that reads them. The vector work hides
// behind the matrix pipe (an 8-pass MFMA leaves seven issue slots) and LDS carries 4 bytes per element instead of 6.
template <int R, bool KC, int NT, int BKD>
struct SplitFrag {
  using D = DirectTile<R, KC, NT, BKD>;
  __device__ static __forceinline__ void load(const float *lds, int row, int c, int g, float (&x)[8]) {
    if (KC) {
      const v4f lo = *reinterpret_cast<const v4f *>(lds + row * BKD + 4 * ((4 * c + 2 * g) ^ D::sw(row)));
      const v4f hi = *reinterpret_cast<const v4f *>(lds + row * BKD + 4 * ((4 * c + 2 * g + 1) ^ D::sw(row)));
#pragma unroll
      for (int i = 0; i < 4; i++) { x[i] = lo[i]; x[4 + i] = hi[i]; }
    } else {
      const float *q = lds + (16 * c + 8 * g) * R + row;
#pragma unroll
      for (int i = 0; i < 8; i++) x[i] = q[i * R];
    }
  }
};

// The pieces (na, nb) of one step's inputs (xa, xb)
template <int TM, int TN>
__device__ __forceinline__ void split_cut(const float (&xa)[TM][8], const float (&xb)[TN][8], v4u (&na)[TM][3], v4u (&nb)[TN][3]) {
#pragma unroll
  for (int q = 0; q < (TM + TN) * 4; q++) {
    const int f = q / 4, p = q % 4;
    unsigned h, m, l;
    if (f < TM) {
      split_pair(xa[f][2 * p], xa[f][2 * p + 1], h, m, l);
      na[f][0][p] = h; na[f][1][p] = m; na[f][2][p] = l;
    } else {
      split_pair(xb[f - TM][2 * p], xb[f - TM][2 * p + 1], h, m, l);
      nb[f - TM][0][p] = h; nb[f - TM][1][p] = m; nb[f - TM][2][p] = l;
    }
  }
}

// One 16-deep step: the TM x TN x 6 MFMAs of the pieces in (fa, fb), smallest terms first, and between them, in
// program order that the scheduler may not change, the cutting of the next step's inputs (xa, xb) into (na, nb):
// (TM + TN) x 4 pairs of elements, 11 vector instructions a pair, dealt evenly over the MFMAs.
template <int TM, int TN>
__device__ __forceinline__ void split_step(const v4u (&fa)[TM][3], const v4u (&fb)[TN][3], v16f (&acc)[TM][TN], const float (&xa)[TM][8],
                                           const float (&xb)[TN][8], v4u (&na)[TM][3], v4u (&nb)[TN][3]) {
  constexpr int TERM_A[6] = {0, 2, 1, 0, 1, 0}, TERM_B[6] = {2, 0, 1, 1, 0, 0};
  constexpr int NMMA = TM * TN * 6, NPAIR = (TM + TN) * 4;
#pragma unroll
  for (int n = 0; n < NMMA; n++) {
    const int t = n / (TM * TN), i = (n / TN) % TM, j = n % TN;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, fb[j][TERM_B[t]]), __builtin_bit_cast(v8bf, fa[i][TERM_A[t]]),
                                                        acc[i][j], 0, 0, 0);   // C^T tile
#pragma unroll
    for (int q = n * NPAIR / NMMA; q < (n + 1) * NPAIR / NMMA; q++) {
      const int f = q / 4, p = q % 4;
      unsigned h, m, l;
      if (f < TM) {
        split_pair(xa[f][2 * p], xa[f][2 * p + 1], h, m, l);
        na[f][0][p] = h; na[f][1][p] = m; na[f][2][p] = l;
      } else {
        split_pair(xb[f - TM][2 * p], xb[f - TM][2 * p + 1], h, m, l);
        nb[f - TM][0][p] = h; nb[f - TM][1][p] = m; nb[f - TM][2][p] = l;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // the pieces exist here, among the MFMAs, not where the next step first reads them (the compiler would sink their computation there)
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int p = 0; p < 3; p++) asm volatile("" : "+v"(na[i][p]));
#pragma unroll
  for (int j = 0; j < TN; j++)
#pragma unroll
    for (int p = 0; p < 3; p++) asm volatile("" : "+v"(nb[j][p]));
}

// The work of one workgroup on output tile (pm, pn) and K split or batch member z
template <int BM, int BN, int WM, int WN, int KIND, int BK, int NSTG, bool SEG2, bool BAND = false, bool MSEG = false, bool SPLIT = false>
__device__ __forceinline__ void gemm_direct_tile(const GemmArgs &a, const int pm, const int pn, const int z) {
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  using TA = DirectTile<BM, KIND != GT_TN, NT, BK>;
  using TB = DirectTile<BN, KIND == GT_NT, NT, BK>;
  extern __shared__ __attribute__((aligned(16))) float smem[];   // [NSTG][A tile | B tile]
  constexpr int STAGE = (TA::CH + TB::CH) * 4;                // floats per stage
  if (a.M < 0) smem[threadIdx.x] = 0.f;                       // never taken: keeps the LDS array "written" for the compiler

  const int m0 = pm * BM, n0 = pn * BN;
  const float *A = a.A, *B = a.B;
  int k0 = 0, kend = a.K;
  if (BAND) {
    // A is kept in blocks: [z][row tile of 128][k step of 32][128 rows][32 k], one contiguous 16 KB block per stage
    static_assert(!BAND || (BM == 128 && BK == 32), "banded A blocks are 128 rows x 32 k");
    A += z * a.sA + (size_t)pm * (a.K / 32) * 4096;
    B += (z / a.zdiv) * a.sB + ((z % a.zdiv) / a.zgroup) * a.sB2;
    k0 = a.window > 0 ? (max(0, m0 - a.window + 1) & ~127) : 0;
    kend = min(a.K, m0 + BM);
    if (a.splits > 1) {                       // this workgroup's share of the row tile's stages (possibly none: it then writes zeros)
      const int nst = (kend - k0) / BK, per = (nst + a.splits - 1) / a.splits;
      k0 = min(kend, k0 + (int)blockIdx.y * per * BK);
      kend = min(kend, k0 + per * BK);
    }
  } else if (a.splits > 1) { k0 = z * a.kchunk; kend = min(a.K, k0 + a.kchunk); }
  else { A += z * a.sA; B += z * a.sB; }
  // The wavefront's index as a scalar for the loads (which of a stage's loads are its own, and their LDS addresses, are then
  // scalar arithmetic instead of vector instructions among the MFMAs); its part of the tile stays derived from the thread
  // index (with a scalar there the 4 x 1 wave layouts ran 10-20 % slower). Measured exception: the NN product on the 4 x 1
  // layout at K = 1536 loses 9 % with the scalar form (its seven loads then leave in one burst) and keeps the vector one.
  constexpr bool SCALAR_WAVE = !(KIND == GT_NN && WN == 1);
  const int tid = threadIdx.x, lane = tid % 64, wave = SCALAR_WAVE ? __builtin_amdgcn_readfirstlane(tid / 64) : tid / 64;
  const int wm = (tid / 64) / WN, wn = (tid / 64) % WN;
  const int g = lane / 32, l32 = lane % 32;

  // wave-uniform source of the next stage to issue (bytes), and this lane's fixed offsets from it
  const char *ba = reinterpret_cast<const char *>(BAND ? A + (size_t)(k0 / BK) * 4096
                                                       : TA::origin(A, a.lda, m0) + (size_t)(k0 / BK) * TA::stage_step(a.lda));
  const char *bb = reinterpret_cast<const char *>(TB::origin(B, a.ldb, n0) + (size_t)(k0 / BK) * TB::stage_step(a.ldb));
  unsigned oa[TA::PER], ob[TB::PER];
#pragma unroll
  for (int i = 0; i < TA::PER; i++) oa[i] = BAND ? TA::off(32, 0, BM, wave, i, lane) : TA::off(a.lda, m0, a.M, wave, i, lane);
#pragma unroll
  for (int i = 0; i < TB::PER; i++) ob[i] = TB::off(a.ldb, n0, a.N, wave, i, lane);
  size_t sta = (BAND ? (size_t)4096 : TA::stage_step(a.lda)) * sizeof(float), stb = TB::stage_step(a.ldb) * sizeof(float);
  // MSEG: stages of the current segment still to be issued, and the segment after it (wave-uniform)
  int seg_left = MSEG ? a.K / BK : 0, seg_next = 0;
#define ISSUE(buf_)                                                                                              \
  {                                                                                                              \
    float *sa_ = smem + (buf_) * STAGE, *sb_ = sa_ + TA::CH * 4;                                                 \
    _Pragma("unroll") for (int i = 0; i < TA::PER; i++) {                                                        \
      asm volatile("" : "+v"(oa[i]));  /* keeps the offset a 32-bit register: scalar base + lane offset */        \
      load_to_lds16(reinterpret_cast<const float *>(ba + oa[i]), sa_ + TA::load_index(wave, i) * 256);           \
    }                                                                                                            \
    _Pragma("unroll") for (int i = 0; i < TB::PER; i++) {                                                        \
      asm volatile("" : "+v"(ob[i]));                                                                            \
      load_to_lds16(reinterpret_cast<const float *>(bb + ob[i]), sb_ + TB::load_index(wave, i) * 256);           \
    }                                                                                                            \
    ba += sta; bb += stb;                                                                                        \
  }
  // the stage of the second segment (SEG2): its sources are computed when it is issued, once per workgroup
#define ISSUE2(buf_)                                                                                             \
  {                                                                                                              \
    float *sa_ = smem + (buf_) * STAGE, *sb_ = sa_ + TA::CH * 4;                                                 \
    _Pragma("unroll") for (int i = 0; i < TA::PER; i++)                                                          \
      load_to_lds16(TA::src2(a.A2, a.lda2, m0, a.M, a.K2, wave, i, lane), sa_ + TA::load_index(wave, i) * 256);  \
    _Pragma("unroll") for (int i = 0; i < TB::PER; i++)                                                          \
      load_to_lds16(TB::src2(a.B2, a.ldb2, n0, a.N, a.K2, wave, i, lane), sb_ + TB::load_index(wave, i) * 256);  \
  }
  // a further segment starts: this lane's sources move to its operands (once per segment and workgroup)
#define NEXT_SEGMENT()                                                                                           \
  {                                                                                                              \
    const float *A_ = a.xA[seg_next], *B_ = a.xB[seg_next];                                                      \
    const int lda_ = a.xlda[seg_next], ldb_ = a.xldb[seg_next];                                                  \
    ba = reinterpret_cast<const char *>(TA::origin(A_, lda_, m0));                                               \
    bb = reinterpret_cast<const char *>(TB::origin(B_, ldb_, n0));                                               \
    _Pragma("unroll") for (int i = 0; i < TA::PER; i++) oa[i] = TA::off(lda_, m0, a.M, wave, i, lane);           \
    _Pragma("unroll") for (int i = 0; i < TB::PER; i++) ob[i] = TB::off(ldb_, n0, a.N, wave, i, lane);           \
    sta = TA::stage_step(lda_) * sizeof(float); stb = TB::stage_step(ldb_) * sizeof(float);                      \
    seg_left = a.xK[seg_next] / BK; seg_next++;                                                                  \
  }
#define ISSUE_STAGE(buf_, st_)                                                                                   \
  {                                                                                                              \
    if (MSEG) { if (seg_left == 0) NEXT_SEGMENT() seg_left--; }                                                  \
    if (SEG2 && (st_) == nstage - 1) ISSUE2(buf_) else ISSUE(buf_)                                               \
  }

  v16f acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // Ring of NSTG stages. Step k: wait until this wavefront's loads of stage k have landed (the younger stages may
  // still be in flight), barrier (every wavefront's part of stage k is there, and everybody is done reading the
  // buffer of stage k-1), issue stage k+NSTG-1 into that buffer, compute stage k.
  constexpr int LPS = TA::PER + TB::PER;                      // loads per wavefront and stage
  constexpr int INFLIGHT = (NSTG - 2) * LPS;                  // loads that may be outstanding when stage k is needed
  static_assert(INFLIGHT < 64, "vmcnt holds six bits");
  int nstage = (kend - k0) / BK + (SEG2 ? 1 : 0);
  if (MSEG) for (int i = 0; i < a.nx; i++) nstage += a.xK[i] / BK;
#pragma unroll
  for (int st = 0; st < NSTG - 1; st++)
    if (st < nstage) ISSUE_STAGE(st, st)
  if constexpr (SPLIT) {
    // The K loop as a chain of 16-deep steps, two per stage. While the MFMAs of one step issue (six per pair of blocks,
    // smallest terms first), the inputs of the next step are cut into their pieces: an 8-pass MFMA leaves seven issue slots, and
    // the order below is forced on the scheduler so that every MFMA is followed by its share of that vector work. The barrier
    // sits between a stage's two steps: by then every wavefront has the stage's second half in registers, so the stage's
    // buffer is free for the stage after next, and the next stage (issued a stage ago) is what the second step prepares from.
    static_assert(!SPLIT || (BK == 32 && NSTG == 2), "two 16-deep steps per stage, two stages");
    using SA = SplitFrag<BM, KIND != GT_TN, NT, BK>;
    using SB = SplitFrag<BN, KIND == GT_NT, NT, BK>;
    v4u f0a[TM][3], f0b[TN][3], f1a[TM][3], f1b[TN][3];
    float xa[TM][8], xb[TN][8];
    const int rowa = wm * (TM * 32) + l32, rowb = wn * (TN * 32) + l32;
#define RAW(sa_, sb_, c_)                                                                              \
  {                                                                                                    \
    _Pragma("unroll") for (int i = 0; i < TM; i++) SA::load(sa_, rowa + i * 32, c_, g, xa[i]);         \
    _Pragma("unroll") for (int j = 0; j < TN; j++) SB::load(sb_, rowb + j * 32, c_, g, xb[j]);         \
  }
    if (nstage > 0) {
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __syncthreads();
      if (1 < nstage) ISSUE_STAGE(1, 1)
      RAW(smem, smem + TA::CH * 4, 0)
      split_cut<TM, TN>(xa, xb, f0a, f0b);          // the first step's inputs, with nothing to multiply yet
      int buf = 0;
      for (int st = 0; st < nstage; st++) {
        const float *sa = smem + buf * STAGE, *sb = sa + TA::CH * 4;
        RAW(sa, sb, 1)
        split_step<TM, TN>(f0a, f0b, acc, xa, xb, f1a, f1b);
        if (SEG2 && st == nstage - 1 && a.K2 <= 16) {
          // a second segment of 16 fills half of its stage: the other half (valid chunks loaded again) is multiplied by zeros
#pragma unroll
          for (int j = 0; j < TN; j++)
#pragma unroll
            for (int p = 0; p < 3; p++) f1b[j][p] = v4u{0, 0, 0, 0};
        }
        // (after the last stage this prepares a step nobody multiplies, from the other buffer's old contents)
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (st + 2 < nstage) ISSUE_STAGE(buf, st + 2)
        const float *na = smem + (buf ^ 1) * STAGE, *nb = na + TA::CH * 4;
        RAW(na, nb, 0)
        split_step<TM, TN>(f1a, f1b, acc, xa, xb, f0a, f0b);
        buf ^= 1;
      }
    }
#undef RAW
  } else {
  int buf = 0;
  for (int st = 0; st < nstage; st++) {
    // vmcnt(n): bits 3:0 and 15:14 of the immediate; the other counters are left at "no wait"
    if (st + NSTG - 2 < nstage) __builtin_amdgcn_s_waitcnt(0x0F70 | (INFLIGHT & 15) | ((INFLIGHT >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0x0F70);                  // the tail: fewer stages are in flight than INFLIGHT assumes
    __syncthreads();
    if (st + NSTG - 1 < nstage) { const int nb = (buf + NSTG - 1) % NSTG; ISSUE_STAGE(nb, st + NSTG - 1) }
    const float *sa = smem + buf * STAGE, *sb = sa + TA::CH * 4;
    const int nrun = (SEG2 && st == nstage - 1) ? a.K2 / 8 : BK / 8;      // the second segment fills its stage partly
#pragma unroll
    for (int c = 0; c < BK / 8; c++) {
      if (!SEG2 || c < nrun) {                                             // wave-uniform
        v4f fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; i++) fa[i] = TA::fetch(sa, wm * (TM * 32) + i * 32 + l32, c, g);
#pragma unroll
        for (int j = 0; j < TN; j++) fb[j] = TB::fetch(sb, wn * (TN * 32) + j * 32 + l32, c, g);
#pragma unroll
        for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
          for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j][s4], fa[i][s4], acc[i][j], 0, 0, 0);   // C^T tile
      }
    }
    buf = (buf + 1) % NSTG;
  }
  }
#undef ISSUE_STAGE
#undef NEXT_SEGMENT
#undef ISSUE2
#undef ISSUE

  float *C;
  int ldc;
  bool add;
  if (BAND) {
    C = (a.splits > 1 ? a.Pp + (size_t)blockIdx.y * a.sP : a.C) + (z / a.zdiv) * a.sC + (z % a.zdiv) * a.sC2;
    ldc = a.ldc;
    add = a.splits > 1 ? false : a.acc != 0;
  }
  else if (a.splits > 1) { C = a.Pp + (size_t)z * a.M * a.N; ldc = a.N; add = false; }
  else { C = a.C + z * a.sC; ldc = a.ldc; add = a.acc != 0 || a.D != nullptr; }
  const float *Cold = (!BAND && a.D && a.splits == 1) ? a.D + z * a.sD : C;
  const bool scaled = !BAND && a.scaled && a.splits == 1;
  // The MFMAs above take the B tile as their first operand, so an accumulator holds a C^T tile: lane l32 is the row
  // of C, and registers 4q..4q+3 are four consecutive columns 8q + 4g + (0..3): one 16-byte store (and, when
  // accumulating, one 16-byte load issued before any store) instead of four scalar ones.
  const bool vec_c = (ldc % 4 == 0) && (((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(Cold)) & 15) == 0);
  if constexpr (BAND) {
    if (a.rope && a.splits == 1) {
      // dQ with respect to the rows before their rotation: a pair (j, j + BN/2) of a row sits in two wavefronts' accumulators
      // (WN = 2), so the tile goes through LDS once (the pipeline's buffers are idle now) and every thread then rotates
      // float4 pairs of whole rows: (lo, hi) -> (c lo + s hi, -s lo + c hi), the reference's srcRope backward (wgsl.ts:346-384)
      // (the launchers size the dynamic LDS for the larger of the pipeline and this tile: band_lds_bytes)
      constexpr int LDS_C = BN + 4;            // = 4 mod 32 words: 8 lanes of a b128 access cover all banks
      __syncthreads();                         // everybody is done reading the last stage
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int q = 0; q < 4; q++)
            *reinterpret_cast<v4f *>(smem + (wm * (TM * 32) + i * 32 + l32) * LDS_C + wn * (TN * 32) + j * 32 + 8 * q + 4 * g) =
                v4f{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
      __syncthreads();
      constexpr int UPR = BN / 8;              // float4 pairs per row
      for (int u = tid; u < BM * UPR; u += NT) {
        const int rl = u / UPR, c = 4 * (u % UPR), row = m0 + rl;
        const v4f lo = *reinterpret_cast<const v4f *>(smem + rl * LDS_C + c), hi = *reinterpret_cast<const v4f *>(smem + rl * LDS_C + BN / 2 + c);
        const float *tp = a.rope + ((size_t)row * (BN / 2) + c) * 2;
        const v4f c0 = *reinterpret_cast<const v4f *>(tp), c1 = *reinterpret_cast<const v4f *>(tp + 4);
        const v4f cs = {c0[0], c0[2], c1[0], c1[2]}, sn = {c0[1], c0[3], c1[1], c1[3]};
        float *cr = C + (size_t)row * ldc + c;
        v4f r0 = cs * lo + sn * hi, r1 = -sn * lo + cs * hi;
        if (add) { r0 += *reinterpret_cast<const v4f *>(cr); r1 += *reinterpret_cast<const v4f *>(cr + BN / 2); }
        if (row < a.M) {
          *reinterpret_cast<v4f *>(cr) = r0;
          *reinterpret_cast<v4f *>(cr + BN / 2) = r1;
        }
      }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      const int row = m0 + wm * (TM * 32) + i * 32 + l32;
      const int cbase = n0 + wn * (TN * 32) + j * 32 + 4 * g;
      if (vec_c) {
        v4f old[4];
        if (add) {
          const float *cr = Cold + (size_t)min(row, a.M - 1) * ldc;
#pragma unroll
          for (int q = 0; q < 4; q++) old[q] = *reinterpret_cast<const v4f *>(cr + min(cbase + 8 * q, a.N - 4));
        }
        if (row >= a.M) continue;
        float *cr = C + (size_t)row * ldc;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int col = cbase + 8 * q;
          if (col >= a.N) continue;                       // N is a multiple of 4 here: a chunk is all in or all out
          v4f o = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
          if (add) o = scaled ? a.dscale * old[q] + a.pscale * o : o + old[q];
          *reinterpret_cast<v4f *>(cr + col) = o;
        }
      } else {
        if (row >= a.M) continue;
        float *cr = C + (size_t)row * ldc;
        float old[16];
        if (add) {
          const float *co = Cold + (size_t)row * ldc;
#pragma unroll
          for (int r = 0; r < 16; r++) old[r] = co[min(cbase + 8 * (r / 4) + (r % 4), a.N - 1)];
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int col = cbase + 8 * (r / 4) + (r % 4);
          if (col < a.N) cr[col] = !add ? acc[i][j][r] : scaled ? a.dscale * old[r] + a.pscale * acc[i][j][r] : old[r] + acc[i][j][r];
        }
      }
    }
}

template <int BM, int BN, int WM, int WN, int KIND, int BK, int NSTG, bool SEG2, bool BAND = false, bool MSEG = false, bool SPLIT = false>
__global__ __launch_bounds__(WM *WN * 64) void gemm_direct(GemmArgs a) {
  int pm, pn, z;
  if (BAND) {
    // Row tiles differ in K range (128 ... T keys). The grid is (batch members, 1, row tiles): dispatch order runs over
    // the batch members of the longest row tile first, then the next shorter one, so the long workgroups start first and
    // the short ones fill the gaps at the end, and the 8 XCDs (fed round-robin in dispatch order) get equal lengths.
    z = blockIdx.x;
    pn = blockIdx.z % a.nbn;
    pm = a.nbm - 1 - (int)(blockIdx.z / a.nbn);
  } else {
    tile_of_workgroup(a, pm, pn, z);
  }
  gemm_direct_tile<BM, BN, WM, WN, KIND, BK, NSTG, SEG2, BAND, MSEG, SPLIT>(a, pm, pn, z);
}

// Several independent TN products with the same K in one launch: the weight gradients dW_i = dY_i^T . X_i of consecutive
// linears of a layer, whose outputs are too small to fill the chip one at a time. The output tiles of all problems form
// one list (problem after problem, N fastest inside a problem); with K splits the (split, tile) pairs are numbered
// split-major and dealt to the XCDs in contiguous ranges, exactly as for a single product. A workgroup looks up its
// problem, points the argument block at that problem's operands, and runs the ordinary tile loop.
#define GT_GROUP_MAX 8
#define GT_DIRECT_LD_MAX (1 << 22)     // largest leading dimension (floats) the direct kernels address: 192 rows x 4 B x this < 2^32
struct GroupProb { const float *A, *B; float *C; int M, N, acc, tile0, nbn; int64_t e0; };   // e0: elements of the problems before it
struct GroupArgs { GroupProb p[GT_GROUP_MAX]; int n, ntiles; };

template <int BM, int BN, int WM, int WN, int BK, int NSTG, bool SPLIT = false>
__global__ __launch_bounds__(WM *WN * 64) void gemm_group_tn(GemmArgs a, GroupArgs g) {
  const int total = g.ntiles * a.splits, lin = blockIdx.x;
  const int xcd = lin % 8, idx = lin / 8, base = total / 8, rem = total % 8;
  const int w = xcd * base + (xcd < rem ? xcd : rem) + idx;
  const int z = w / g.ntiles, pid = w % g.ntiles;
  int i = 0;
#pragma unroll
  for (int q = 1; q < GT_GROUP_MAX; q++) if (q < g.n && pid >= g.p[q].tile0) i = q;
  const GroupProb &p = g.p[i];
  const int lp = pid - p.tile0;
  a.A = p.A; a.B = p.B; a.C = p.C;
  a.M = p.M; a.N = p.N; a.lda = p.M; a.ldb = p.N; a.ldc = p.N; a.acc = p.acc;
  a.Pp += (size_t)a.splits * p.e0;
  gemm_direct_tile<BM, BN, WM, WN, GT_TN, BK, NSTG, false, false, false, SPLIT>(a, lp / p.nbn, lp % p.nbn, z);
}

// dynamic LDS of a banded launch: the pipeline's stages, or the BM x (BN + 4) tile its rotating write-back passes through LDS
template <int BM, int BN, int BK, int NSTG>
constexpr int band_lds_bytes() {
  return 4 * (NSTG * (BM + BN) * BK > BM * (BN + 4) ? NSTG * (BM + BN) * BK : BM * (BN + 4));
}


// gemm_split.hip: the bf16-piece instantiations. wide: 128 x 192 tiles (N a multiple of 192), else 128 x 128; summed: the
// argument block carries further K segments (gt_gemm_sum).
int gemm_split_launch(gt_ctx *ctx, int kind, bool wide, bool summed, GemmArgs &a, int zdim);
int gemm_split_launch_group(gt_ctx *ctx, bool wide, GemmArgs &a, GroupArgs &g);
// the banded batch (dQ = dS.K per (sequence, head), head dim 64): 128 x 64 tiles, two wavefronts of 64 x 64
int gemm_split_launch_band(gt_ctx *ctx, GemmArgs &a, int zdim);
