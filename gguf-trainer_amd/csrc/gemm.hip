// FP32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32), the contraction behind
// linear forward (NT), dX = dY.W (NN) and dW = dY^T.X (TN), the chunked-CE readout and the
// Newton-Schulz products. Replaces srcGemm (src/backend/wgsl.ts:87-196).
//
// Two kernels share the tile shapes and the epilogue. gemm_direct (aligned shapes: K a multiple of 32, whole 16-byte
// chunks along every operand's contiguous index) brings operand tiles from global memory straight into LDS, double
// buffered, one barrier per K step; it is described where it is defined. gemm_kernel, described here, stages them
// through registers and takes every shape (two-segment products with a long or odd second segment included).
//
// Shape of the kernel. A workgroup of WM x WN wavefronts owns a BM x BN tile of C and walks K in
// steps of 16 or 32. Each wavefront owns a (BM/WM) x (BN/WN) sub-tile as TM x TN MFMA tiles of 32x32,
// 16 accumulator VGPRs each. Global loads for step i+1 are issued into registers before the
// MFMAs of step i and stored to LDS after them, so HBM/L2 latency hides under 32+ MFMAs.
//
// LDS layout. Every operand tile is kept as [row][BK+4] so that a lane fetches its MFMA inputs for
// four consecutive steps with one ds_read_b128. An operand whose K index is contiguous in memory
// (A of NT/NN, B of NT) is copied float4 for float4; one whose row index is contiguous (A of TN,
// B of NN/TN) is transposed on the way in (see Tile). Because an MFMA step consumes K pairs
// (lane/32 selects which), the order in which K is consumed is free as long as A and B agree:
// inside every run of 8, lane group g takes k = 4g + i at step i, which is what lets the b128
// fetch feed four steps.
//
// dW has a small output and a long K (rows of the batch), so it is split along K over blockIdx.z
// into per-split partial tiles in the workspace, summed in split order by a second kernel: no
// atomics, bit-identical from run to run.
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

// The work of one workgroup on output tile (pm, pn) and K split or batch member z
template <int BM, int BN, int WM, int WN, int KIND, int BK, int NSTG, bool SEG2, bool BAND = false, bool MSEG = false>
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
      static_assert(!BAND || NSTG * (BM + BN) * BK >= BM * (BN + 4), "the tile must fit the pipeline's LDS");
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

template <int BM, int BN, int WM, int WN, int KIND, int BK, int NSTG, bool SEG2, bool BAND = false, bool MSEG = false>
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
  gemm_direct_tile<BM, BN, WM, WN, KIND, BK, NSTG, SEG2, BAND, MSEG>(a, pm, pn, z);
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

template <int BM, int BN, int WM, int WN, int BK, int NSTG>
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
  gemm_direct_tile<BM, BN, WM, WN, GT_TN, BK, NSTG, false>(a, lp / p.nbn, lp % p.nbn, z);
}
// C_i (+)= sum over splits of the group's partials, in split order; one thread per output element of the whole group
__global__ __launch_bounds__(256) void group_reduce(GroupArgs g, const float *__restrict__ Pp, int64_t total, int splits) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  int i = 0;
#pragma unroll
  for (int q = 1; q < GT_GROUP_MAX; q++) if (q < g.n && e >= g.p[q].e0) i = q;
  const GroupProb &p = g.p[i];
  const int64_t n = (int64_t)p.M * p.N, l = e - p.e0;
  const float *pp = Pp + (size_t)splits * p.e0 + l;
  float s = pp[0];
  for (int z = 1; z < splits; z++) s += pp[(size_t)z * n];
  p.C[l] = p.acc ? p.C[l] + s : s;
}

template <int BM, int BN, int WM, int WN, int KIND, int BK, int NSTG, bool SEG2>
static int launch_direct_kind(gt_ctx *ctx, GemmArgs &a, int zdim, int slot) {
  constexpr int smem = NSTG * (BM + BN) * BK * 4;
  if (!(ctx->gemm_direct_set & (1ull << slot))) {       // once per context (device): more LDS than a kernel gets by default
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct<BM, BN, WM, WN, KIND, BK, NSTG, SEG2>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_direct_set |= 1ull << slot;
  }
  hipLaunchKernelGGL((gemm_direct<BM, BN, WM, WN, KIND, BK, NSTG, SEG2>), dim3(a.nbm * a.nbn, 1, zdim), dim3(WM * WN * 64), smem, ctx->stream, a);
  GT_LAUNCHED(ctx);
  return 0;
}
// slot: index of the tile shape (0..5); the bit of (shape, kind, one or two segments) in gemm_direct_set follows from it
template <int BM, int BN, int WM, int WN, int BK, int NSTG>
static int launch_direct(gt_ctx *ctx, int kind, GemmArgs &a, int zdim, int slot) {
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  const int b1 = slot < 5 ? 3 * slot : 45 + 3 * (slot - 5), b2 = slot < 5 ? 15 + 2 * slot : 54 + 2 * (slot - 5);
  if (a.K2 > 0) {                // two K segments: NT / NN only
    if (kind == GT_NT) return launch_direct_kind<BM, BN, WM, WN, GT_NT, BK, NSTG, true>(ctx, a, zdim, b2);
    return launch_direct_kind<BM, BN, WM, WN, GT_NN, BK, NSTG, true>(ctx, a, zdim, b2 + 1);
  }
  if (kind == GT_NT) return launch_direct_kind<BM, BN, WM, WN, GT_NT, BK, NSTG, false>(ctx, a, zdim, b1);
  if (kind == GT_NN) return launch_direct_kind<BM, BN, WM, WN, GT_NN, BK, NSTG, false>(ctx, a, zdim, b1 + 1);
  return launch_direct_kind<BM, BN, WM, WN, GT_TN, BK, NSTG, false>(ctx, a, zdim, b1 + 2);
}

// C (+)= sum over splits, in split order
__global__ __launch_bounds__(256) void splitk_reduce(const float *__restrict__ Pp, float *__restrict__ C, int64_t n,
                                                     int splits, int acc, const float *__restrict__ D, int scaled, float dscale,
                                                     float pscale) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = Pp[i];
  for (int z = 1; z < splits; z++) s += Pp[(size_t)z * n + i];
  C[i] = D ? (scaled ? dscale * D[i] + pscale * s : D[i] + s) : acc ? C[i] + s : s;
}

template <int BM, int BN, int WM, int WN, int BKT>
static int launch_cfg(gt_ctx *ctx, int kind, bool vec, GemmArgs &a, int zdim) {
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  dim3 grid(a.nbm * a.nbn, 1, zdim), block(WM * WN * 64);
#define GO(KIND, VEC) hipLaunchKernelGGL((gemm_kernel<BM, BN, WM, WN, BKT, KIND, VEC>), grid, block, 0, ctx->stream, a)
#define GO2(KIND) hipLaunchKernelGGL((gemm_kernel<BM, BN, WM, WN, BKT, KIND, true, true>), grid, block, 0, ctx->stream, a)
  if (a.K2 > 0) {                // two K segments: aligned NT / NN only (gemm_impl sends everything else as two launches)
    if (kind == GT_NT) GO2(GT_NT); else GO2(GT_NN);
  }
  else if (kind == GT_NT) { if (vec) GO(GT_NT, true); else GO(GT_NT, false); }
  else if (kind == GT_NN) { if (vec) GO(GT_NN, true); else GO(GT_NN, false); }
  else { if (vec) GO(GT_TN, true); else GO(GT_TN, false); }
#undef GO2
#undef GO
  GT_LAUNCHED(ctx);
  return 0;
}

static int reduce_splits(gt_ctx *ctx, const GemmArgs &a, int M, int N, int splits, int acc) {
  if (splits > 1) {
    int64_t n = (int64_t)M * N;
    hipLaunchKernelGGL(splitk_reduce, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, ctx->stream, a.Pp, a.C, n, splits, acc, a.D, a.scaled, a.dscale, a.pscale);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

struct TileCfg { int bm, bn, bk; };
static const TileCfg kTiles[] = {{64, 64, 16}, {128, 64, 16}, {128, 128, 16}, {128, 192, 16}, {128, 96, 16}, {256, 128, 16},
                                 {128, 128, 32}, {128, 192, 32}, {128, 96, 32}, {256, 128, 32}, {64, 192, 16}, {128, 64, 32}, {64, 192, 32}, {128, 160, 32}};
#define NCFG ((int)(sizeof(kTiles) / sizeof(kTiles[0])))

// Tile and split-K choice by a small cost model over the tile shapes that measured best on MI355X:
// time ~ flops / (tile efficiency x edge utilisation x wave quantisation) + the cost of the split-K reduction pass,
// for one product (batched `count` times) or a group of `np` products with a common K launched together.
struct Cand { int cfg; double eff; };
static void pick_tile(gt_ctx *ctx, int kind, bool direct_ok, int np, const int *Ms, const int *Ns, int K, int count, bool two_seg,
                      int *cfg_out, int *splits_out, int fixed_splits = 0) {
  // relative tile efficiencies as measured (asymptotic rate of each tile over the best one's)
  static const Cand cand_nn[] = {{7, 1.00}, {6, 0.98}, {8, 0.98}, {10, 0.95}, {11, 0.82}, {0, 0.78}};
  static const Cand cand_tn[] = {{8, 1.00}, {11, 0.99}, {10, 0.92}, {6, 0.90}, {7, 0.78}, {0, 0.72}};
  static const Cand cand_nn_direct[] = {{7, 1.00}, {8, 1.00}, {13, 1.00}, {6, 0.98}, {12, 0.97}, {11, 0.92}, {10, 0.85}, {0, 0.72}};
  static const Cand cand_tn_direct[] = {{8, 1.00}, {12, 1.00}, {13, 0.99}, {7, 0.98}, {11, 0.96}, {6, 0.88}, {10, 0.85}, {0, 0.68}};
  const Cand *cand = direct_ok ? (kind == GT_TN ? cand_tn_direct : cand_nn_direct) : (kind == GT_TN ? cand_tn : cand_nn);
  const int ncand = direct_ok ? 8 : 6;
  int cfg = 0, splits = 1;
  double elems = 0;
  for (int i = 0; i < np; i++) elems += (double)Ms[i] * Ns[i];
  const double flops = 2.0 * elems * K * count;
  const double t0 = flops / (direct_ok ? 132e12 : 125e12);   // seconds at the best tile's asymptotic rate
  double best = 1e30;
  for (int ci = 0; ci < ncand; ci++) {
    const Cand &c = cand[ci];
    const TileCfg &tc = kTiles[c.cfg];
    if (np > 1 && !(c.cfg == 6 || c.cfg == 7 || c.cfg == 8 || c.cfg == 11 || c.cfg == 12 || c.cfg == 13)) continue;   // group launches: direct tiles only
    int64_t tiles = 0;
    for (int i = 0; i < np; i++) tiles += cdiv(Ms[i], tc.bm) * cdiv(Ns[i], tc.bn);
    const double util = elems / ((double)tiles * tc.bm * tc.bn);
    // any split count, not only powers of two: 72 output tiles x 14 splits is 3.94 workgroups per CU, x 16 is 4.5,
    // and with workgroups of equal length the CUs that get the fifth one set the time
    for (int sp = fixed_splits > 0 ? fixed_splits : 1; sp <= (fixed_splits > 0 ? fixed_splits : 64); sp++) {
      // split only when the output tiles alone cannot give every CU a workgroup (a group's split count is given)
      if (!fixed_splits && sp > 1 && (count > 1 || two_seg || tiles >= ctx->num_cu || K / sp < 8 * tc.bk)) break;
      const double waves = (double)tiles * sp * count / ctx->num_cu;
      const double quant = waves / ceil(waves);
      // a CU with few workgroups over the whole launch overlaps their fills and write-backs less (fitted on the
      // dW shapes: 1 workgroup per CU runs 15 % and 2 run 6 % below the rate reached from 4 per CU on)
      const double conc = std::min(1.0, 1.0625 * waves / (waves + 0.25));
      // short K per workgroup pays the prologue/epilogue more: ~2 K-steps of overhead
      const double ksteps = (double)K / sp / tc.bk;
      const double depth = ksteps / (ksteps + 2.0);
      double t = t0 / (c.eff * util * quant * depth * conc);
      if (sp > 1) t += ((double)(sp + 2) * elems * 4.0) / 3.5e12 + 4e-6;
      if (t < best) { best = t; cfg = c.cfg; splits = sp; }
    }
  }
  *cfg_out = cfg;
  *splits_out = splits;
}

static int gemm_impl(gt_ctx *ctx, int kind, int acc, int M, int N, int K, gt_buf A, int64_t sA, gt_buf B, int64_t sB,
                     gt_buf C, int64_t sC, int count, int K2 = 0, gt_buf A2 = 0, gt_buf B2 = 0, gt_buf D = 0, int64_t sD = 0,
                     int scaled = 0, float dscale = 1.f, float pscale = 1.f) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, kind >= 0 && kind <= 2, "gt_gemm: kind %d is not NT(0)/NN(1)/TN(2)", kind);
  GT_REQUIRE(ctx, M >= 1 && N >= 1 && K >= 1 && count >= 1, "gt_gemm: M,N,K,count must be >= 1 (got %d,%d,%d,%d)", M, N, K, count);
  GT_REQUIRE(ctx, A && B && C, "gt_gemm: null operand");
  GemmArgs a;
  a.A = P<const float>(A); a.B = P<const float>(B); a.C = P<float>(C);
  a.M = M; a.N = N; a.K = K;
  a.lda = (kind == GT_TN) ? M : K;
  a.ldb = (kind == GT_NT) ? K : N;
  a.ldc = N;
  a.acc = acc; a.kchunk = K; a.splits = 1; a.Pp = nullptr;
  a.sA = sA; a.sB = sB; a.sC = sC;
  a.zdiv = a.zgroup = 1; a.window = 0; a.sB2 = a.sC2 = 0; a.nx = 0; a.D = P<const float>(D);
  a.sD = sD; a.scaled = scaled; a.dscale = dscale; a.pscale = pscale; a.rope = nullptr;
  GT_REQUIRE(ctx, !D || K2 == 0, "gt_gemm_add: single-segment products only");
  GT_REQUIRE(ctx, !scaled || D, "scaled write-back needs the matrix it combines the product with");
  bool vec = (a.lda % 4 == 0) && (a.ldb % 4 == 0) && (A % 16 == 0) && (B % 16 == 0) &&
             (sA % 4 == 0) && (sB % 4 == 0);
  a.K2 = K2; a.A2 = P<const float>(A2); a.B2 = P<const float>(B2);
  a.lda2 = (kind == GT_TN) ? M : K2;
  a.ldb2 = (kind == GT_NT) ? K2 : N;
  if (K2 > 0) vec = vec && (a.lda2 % 4 == 0) && (a.ldb2 % 4 == 0) && (A2 % 16 == 0) && (B2 % 16 == 0);

  // Tile and split-K choice: pick_tile. N = 576 (SmolLM2) is 3x192 = 6x96; dW has a 1536x576 output and
  // K = 16384 rows, which only fills 256 CUs when K is split.
  // Tiles with a K step of 32 have a variant that loads operands straight into LDS (gemm_direct); it wants whole K
  // steps and whole 16-byte chunks along the contiguous index of every operand. Where it applies it is 2-8 % faster
  // than the register-staged kernel of the same tile and changes which tile is best, hence two tables.
  // a lane's byte offset inside a tile (up to 192 rows of ld floats) must fit the 32 bits the direct kernels keep it in
  const bool direct_ok = vec && K % 32 == 0 && (kind != GT_TN || (M % 4 == 0 && M >= 4)) && (kind == GT_NT || (N % 4 == 0 && N >= 4)) &&
                         std::max(std::max(a.lda, a.ldb), K2 > 0 ? std::max(a.lda2, a.ldb2) : 0) <= GT_DIRECT_LD_MAX &&
                         (K2 == 0 || (kind != GT_TN && K2 % 8 == 0 && K2 <= 32));   // a short second segment rides in one more stage
  int cfg = 0, splits = 1;
  pick_tile(ctx, kind, direct_ok, 1, &M, &N, K, count, K2 > 0, &cfg, &splits);
  if (ctx->opt_gemm_tile >= 0 && ctx->opt_gemm_tile < NCFG) cfg = ctx->opt_gemm_tile;
  const int bm = kTiles[cfg].bm, bn = kTiles[cfg].bn, bk = kTiles[cfg].bk;
  if (count == 1 && K2 == 0 && ctx->opt_gemm_splitk >= 1) splits = ctx->opt_gemm_splitk;
  if (splits > 1) {
    int64_t kc = cdiv(cdiv(K, splits), bk) * bk;
    splits = (int)cdiv(K, kc);
    a.kchunk = (int)kc;
  }
  if (splits > 1) {
    void *ws;
    if (gt_ws_reserve(ctx, (size_t)splits * M * N * sizeof(float), &ws)) return 1;
    a.splits = splits; a.Pp = static_cast<float *>(ws);
  }
  int zdim = splits > 1 ? splits : count;
  char label[32];
  snprintf(label, sizeof label, "gemm.%s.%dx%dx%d%s", kind == GT_NT ? "nt" : kind == GT_NN ? "nn" : "tn", bm, bn, bk, splits > 1 ? ".splitk" : "");
  ProfScope ps(ctx, label, 2.0 * M * N * ((double)K + K2) * count);
  int rc;
  if (direct_ok && !ctx->opt_gemm_staged) {
    switch (cfg) {
      case 6: return launch_direct<128, 128, 2, 2, 32, 2>(ctx, kind, a, zdim, 0) || reduce_splits(ctx, a, M, N, splits, acc);
      case 7: return launch_direct<128, 192, 2, 2, 32, 2>(ctx, kind, a, zdim, 1) || reduce_splits(ctx, a, M, N, splits, acc);
      case 8: return launch_direct<128, 96, 4, 1, 32, 2>(ctx, kind, a, zdim, 2) || reduce_splits(ctx, a, M, N, splits, acc);
      case 11: return launch_direct<128, 64, 2, 2, 32, 2>(ctx, kind, a, zdim, 3) || reduce_splits(ctx, a, M, N, splits, acc);
      case 12: return launch_direct<64, 192, 2, 2, 32, 2>(ctx, kind, a, zdim, 4) || reduce_splits(ctx, a, M, N, splits, acc);
      case 13: return launch_direct<128, 160, 4, 1, 32, 2>(ctx, kind, a, zdim, 5) || reduce_splits(ctx, a, M, N, splits, acc);
      default: break;
    }
  }
  switch (cfg) {
    case 0: rc = launch_cfg<64, 64, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 1: rc = launch_cfg<128, 64, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 2: rc = launch_cfg<128, 128, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 3: rc = launch_cfg<128, 192, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 4: rc = launch_cfg<128, 96, 4, 1, 16>(ctx, kind, vec, a, zdim); break;
    case 5: rc = launch_cfg<256, 128, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 6: rc = launch_cfg<128, 128, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
    case 7: rc = launch_cfg<128, 192, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
    case 8: rc = launch_cfg<128, 96, 4, 1, 32>(ctx, kind, vec, a, zdim); break;
    case 9: rc = launch_cfg<256, 128, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
    case 10: rc = launch_cfg<64, 192, 2, 2, 16>(ctx, kind, vec, a, zdim); break;
    case 11: rc = launch_cfg<128, 64, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
    case 13: rc = launch_cfg<128, 160, 4, 1, 32>(ctx, kind, vec, a, zdim); break;
    default: rc = launch_cfg<64, 192, 2, 2, 32>(ctx, kind, vec, a, zdim); break;
  }
  if (rc) return rc;
  return reduce_splits(ctx, a, M, N, splits, acc);
}

// dQ[b][t][h*hd + :] (+)= sum over the keys s visible from t of dS[b*Hq + h][t][s] * K[b][s][(h/group)*hd + :] for every
// (sequence, head): one banded NN product per pair, all in one launch. dS holds B*Hq [T][T] matrices in blocks
// [row tile of 128][key step of 32][128 rows][32 keys] (what one pipeline stage loads is one contiguous 16 KB block)
// whose blocks inside each row tile's band are all written (zeros where a pair is masked); T is a multiple of 128.
template <int BN>
static int launch_band(gt_ctx *ctx, GemmArgs &a, int zdim, int slot) {
  constexpr int BM = 128, BK = 32, NSTG = 3, WM = 2, WN = 2;
  constexpr int smem = NSTG * (BM + BN) * BK * 4;
  if (!(ctx->gemm_direct_set & (1ull << slot))) {
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct<BM, BN, WM, WN, GT_NN, BK, NSTG, false, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_direct_set |= 1ull << slot;
  }
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  hipLaunchKernelGGL((gemm_direct<BM, BN, WM, WN, GT_NN, BK, NSTG, false, true>), dim3(zdim, a.splits, a.nbm * a.nbn), dim3(WM * WN * 64), smem,
                     ctx->stream, a);
  GT_LAUNCHED(ctx);
  return 0;
}

// dQ (+)= sum of the band product's split partials, in split order, rotated back where the rows are wanted before their
// rotation ((lo, hi) -> (c lo + s hi, -s lo + c hi) per pair (j, j + hd/2), the reference's srcRope backward, wgsl.ts:346-384):
// one thread per float4 of a row's low half and its partner in the high half. rows = B*T rows of Hq heads.
__global__ __launch_bounds__(256) void band_dq_reduce(const float *__restrict__ Pp, int splits, int64_t plane, float *dq, int acc,
                                                      const float *__restrict__ rot, int64_t rows, int T, int Hq, int hd) {
  const int upr = hd / 8;                                  // float4 units in the low half of a head's row
  const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (u >= rows * Hq * upr) return;
  const int c4 = (int)(u % upr);
  const int64_t rh = u / upr, row = rh / Hq;
  const size_t lo = (size_t)rh * hd + 4 * c4, hi = lo + hd / 2;
  v4f a = *reinterpret_cast<const v4f *>(Pp + lo), b = *reinterpret_cast<const v4f *>(Pp + hi);
  for (int z = 1; z < splits; z++) {
    a += *reinterpret_cast<const v4f *>(Pp + (size_t)z * plane + lo);
    b += *reinterpret_cast<const v4f *>(Pp + (size_t)z * plane + hi);
  }
  if (rot) {
    const float *cs = rot + ((size_t)(row % T) * (hd / 2) + 4 * c4) * 2;
    const v4f c0 = *reinterpret_cast<const v4f *>(cs), c1 = *reinterpret_cast<const v4f *>(cs + 4);
    const v4f c = {c0[0], c0[2], c1[0], c1[2]}, sn = {c0[1], c0[3], c1[1], c1[3]};
    const v4f r0 = c * a + sn * b, r1 = -sn * a + c * b;
    a = r0;
    b = r1;
  }
  if (acc) {
    a += *reinterpret_cast<const v4f *>(dq + lo);
    b += *reinterpret_cast<const v4f *>(dq + hi);
  }
  *reinterpret_cast<v4f *>(dq + lo) = a;
  *reinterpret_cast<v4f *>(dq + hi) = b;
}

// how many parts a small launch of the banded product cuts every row tile's K range into (1: none), so that a single
// sequence's 16 row tiles per head, whose longest has 16 times the K range of the shortest, become enough workgroups of
// bounded length to fill the chip; the caller provides that many planes of B*T*Hq*hd floats
int gemm_band_dq_splits(gt_ctx *ctx, int B, int T, int Hq, int window) {
  const int64_t tiles = (int64_t)B * Hq * (T / 128);
  if (ctx->opt_attn_band_splits >= 1) return (int)std::min<int64_t>(std::min(ctx->opt_attn_band_splits, 8), std::max(1, T / 128));
  // the longest K range of a row tile: the whole sequence, or a window's band (there the tiles are short and alike: no cut)
  const int kmax = window > 0 ? std::min(T, ((window + 126) & ~127) + 128) : T;
  if (tiles >= 2 * ctx->num_cu || kmax < 1024) return 1;
  return (int)std::min<int64_t>(std::min<int64_t>(8, kmax / 256), cdiv(2 * ctx->num_cu, tiles));
}

int gemm_band_dq(gt_ctx *ctx, int B, int T, int Hq, int Hkv, int hd, int window, const float *dS, const float *K, float *dQ, int acc,
                 const float *rot, float *parts, int splits) {
  GT_REQUIRE(ctx, T % 128 == 0 && (hd == 64 || hd == 128), "banded dQ product: T %d must be a multiple of 128 and hd %d 64 or 128", T, hd);
  GT_REQUIRE(ctx, ((reinterpret_cast<uintptr_t>(dS) | reinterpret_cast<uintptr_t>(K) | reinterpret_cast<uintptr_t>(dQ)) & 15) == 0,
             "banded dQ product: operands must be 16-byte aligned");
  GemmArgs a;
  a.A = dS; a.B = K; a.C = dQ;
  a.M = T; a.N = hd; a.K = T;
  a.lda = T; a.ldb = Hkv * hd; a.ldc = Hq * hd;
  GT_REQUIRE(ctx, splits >= 1 && (splits == 1 || parts), "banded dQ product: %d splits without a workspace", splits);
  a.acc = acc; a.kchunk = T; a.splits = splits; a.Pp = parts; a.sP = (int64_t)B * T * Hq * hd;
  a.sA = (int64_t)T * T; a.sB = (int64_t)T * Hkv * hd; a.sC = (int64_t)T * Hq * hd;
  a.zdiv = Hq; a.zgroup = Hq / Hkv; a.window = window; a.sB2 = hd; a.sC2 = hd;
  a.A2 = a.B2 = nullptr; a.K2 = 0; a.lda2 = a.ldb2 = 0; a.nx = 0; a.D = nullptr; a.sD = 0; a.scaled = 0; a.dscale = a.pscale = 1.f;
  a.rope = rot;
  GT_REQUIRE(ctx, !rot || (Hq * hd) % 4 == 0, "banded dQ product: rotated rows need 16-byte aligned output rows");
  GT_REQUIRE(ctx, T / 128 <= 65535, "banded dQ product: %d row tiles exceed the grid", T / 128);
  if (hd == 64 ? launch_band<64>(ctx, a, B * Hq, 25) : launch_band<128>(ctx, a, B * Hq, 26)) return 1;
  if (splits > 1) {
    const int64_t rows = (int64_t)B * T, units = rows * Hq * (hd / 8);
    hipLaunchKernelGGL(band_dq_reduce, dim3((unsigned)cdiv(units, 256)), dim3(256), 0, ctx->stream, parts, splits, a.sP, dQ, acc, rot, rows, T, Hq, hd);
    GT_LAUNCHED(ctx);
  }
  return 0;
}

// C (+)= sum over i of A_i.B_i with the K segments chained in one loop (NT / NN, every K_i a multiple of 32)
template <int BM, int BN, int WM, int WN, int KIND>
static int launch_multi(gt_ctx *ctx, GemmArgs &a, int slot) {
  constexpr int BK = 32, NSTG = 2, smem = NSTG * (BM + BN) * BK * 4;
  if (!(ctx->gemm_direct_set & (1ull << slot))) {
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_direct<BM, BN, WM, WN, KIND, BK, NSTG, false, false, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_direct_set |= 1ull << slot;
  }
  a.nbm = (int)cdiv(a.M, BM);
  a.nbn = (int)cdiv(a.N, BN);
  hipLaunchKernelGGL((gemm_direct<BM, BN, WM, WN, KIND, BK, NSTG, false, false, true>), dim3(a.nbm * a.nbn, 1, 1), dim3(WM * WN * 64), smem,
                     ctx->stream, a);
  GT_LAUNCHED(ctx);
  return 0;
}

template <int BM, int BN, int WM, int WN>
static int launch_group(gt_ctx *ctx, GemmArgs &a, GroupArgs &g, int slot) {
  constexpr int BK = 32, NSTG = 2, smem = NSTG * (BM + BN) * BK * 4;
  if (!(ctx->gemm_direct_set & (1ull << slot))) {
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_group_tn<BM, BN, WM, WN, BK, NSTG>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    ctx->gemm_direct_set |= 1ull << slot;
  }
  int tiles = 0;
  for (int i = 0; i < g.n; i++) {
    g.p[i].tile0 = tiles;
    g.p[i].nbn = (int)cdiv(g.p[i].N, BN);
    tiles += (int)cdiv(g.p[i].M, BM) * g.p[i].nbn;
  }
  g.ntiles = tiles;
  hipLaunchKernelGGL((gemm_group_tn<BM, BN, WM, WN, BK, NSTG>), dim3((unsigned)tiles * a.splits), dim3(WM * WN * 64), smem, ctx->stream, a, g);
  GT_LAUNCHED(ctx);
  return 0;
}

extern "C" {
int gt_gemm_group(gt_ctx *ctx, int kind, int count, const int *M, const int *N, int K, const gt_buf *A, const gt_buf *B,
                  const gt_buf *C, const int *acc) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, kind >= 0 && kind <= 2 && count >= 1 && M && N && A && B && C && acc && K >= 1,
             "gt_gemm_group: kind %d, %d products, K %d, or a null table", kind, count, K);
  // What a product's result is, bit for bit, must not depend on which other products it shares a launch with (the host
  // groups what happens to be pending: with and without recomputed regions those are different sets). The tile shape
  // does not enter the arithmetic of an output element (every direct tile walks K in the same order); the K split does.
  // So the split is a function of K alone: ranges of max(512, K/8) rows, at most eight partials per output. A product
  // that fills the chip on its own (at least one 128 x 96 tile per CU) is not split and goes as its own launch.
  const int64_t big = (int64_t)ctx->num_cu * 128 * 96;
  int idx[GT_GROUP_MAX], ng = 0;
  bool eligible = kind == GT_TN && K % 32 == 0 && !ctx->opt_gemm_staged && ctx->opt_gemm_group;      // (TN: ld = M, N, below GT_DIRECT_LD_MAX for any grouped size)
  for (int i = 0; i < count; i++) {
    GT_REQUIRE(ctx, M[i] >= 1 && N[i] >= 1 && A[i] && B[i] && C[i], "gt_gemm_group: product %d has M %d, N %d or a null operand", i, M[i], N[i]);
    for (int j = 0; j < i; j++)
      GT_REQUIRE(ctx, C[i] + (uint64_t)M[i] * N[i] * 4 <= C[j] || C[j] + (uint64_t)M[j] * N[j] * 4 <= C[i],
                 "gt_gemm_group: the outputs of products %d and %d overlap", j, i);
  }
  const int pin = ctx->opt_gemm_tile;
  GT_REQUIRE(ctx, !(eligible && pin >= 0 && pin != 6 && pin != 7 && pin != 8 && pin != 11 && pin != 12 && pin != 13),
             "gt_gemm_group: \"gemm.tile\" pins tile %d, which the grouped launch does not have (6, 7, 8, 11, 12 or 13; -1 = choose)", pin);
  if (count > GT_GROUP_MAX) {
    for (int i = 0; i < count; i += GT_GROUP_MAX)
      if (gt_gemm_group(ctx, kind, std::min(GT_GROUP_MAX, count - i), M + i, N + i, K, A + i, B + i, C + i, acc + i)) return 1;
    return 0;
  }
  for (int i = 0; i < count; i++) {
    const bool fits = eligible && M[i] % 4 == 0 && N[i] % 4 == 0 && (A[i] | B[i] | C[i]) % 16 == 0 && (int64_t)M[i] * N[i] < big &&
                      M[i] <= GT_DIRECT_LD_MAX && N[i] <= GT_DIRECT_LD_MAX;
    if (fits) idx[ng++] = i;
    else if (gemm_impl(ctx, kind, acc[i], M[i], N[i], K, A[i], 0, B[i], 0, C[i], 0, 1)) return 1;
  }
  if (ng == 0) return 0;
  GemmArgs a;
  memset(&a, 0, sizeof a);
  a.K = K; a.kchunk = K; a.splits = 1; a.zdiv = a.zgroup = 1;
  GroupArgs g;
  memset(&g, 0, sizeof g);
  g.n = ng;
  int64_t elems = 0;
  int gm[GT_GROUP_MAX], gn[GT_GROUP_MAX];
  for (int q = 0; q < ng; q++) {
    const int i = idx[q];
    g.p[q].A = P<const float>(A[i]); g.p[q].B = P<const float>(B[i]); g.p[q].C = P<float>(C[i]);
    g.p[q].M = gm[q] = M[i]; g.p[q].N = gn[q] = N[i]; g.p[q].acc = acc[i]; g.p[q].e0 = elems;
    elems += (int64_t)M[i] * N[i];
  }
  int64_t kc = std::max<int64_t>(512, cdiv(cdiv(K, 8), 32) * 32);
  if (ctx->opt_gemm_splitk >= 1) kc = cdiv(cdiv(K, ctx->opt_gemm_splitk), 32) * 32;
  int splits = (int)cdiv(K, kc), cfg = 0, unused = 0;
  pick_tile(ctx, GT_TN, true, ng, gm, gn, K, 1, false, &cfg, &unused, splits);
  if (pin == 6 || pin == 7 || pin == 8 || pin == 11 || pin == 12 || pin == 13) cfg = pin;
  if (splits > 1) {
    a.kchunk = (int)kc;
    void *ws;
    if (gt_ws_reserve(ctx, (size_t)splits * elems * sizeof(float), &ws)) return 1;
    a.splits = splits; a.Pp = static_cast<float *>(ws);
  }
  char label[32];
  snprintf(label, sizeof label, "gemm.tn.group.%dx%d%s", kTiles[cfg].bm, kTiles[cfg].bn, splits > 1 ? ".splitk" : "");
  ProfScope ps(ctx, label, 2.0 * elems * K);
  int rc;
  switch (cfg) {
    case 6: rc = launch_group<128, 128, 2, 2>(ctx, a, g, 40); break;
    case 7: rc = launch_group<128, 192, 2, 2>(ctx, a, g, 41); break;
    case 8: rc = launch_group<128, 96, 4, 1>(ctx, a, g, 42); break;
    case 11: rc = launch_group<128, 64, 2, 2>(ctx, a, g, 43); break;
    case 13: rc = launch_group<128, 160, 4, 1>(ctx, a, g, 58); break;
    default: rc = launch_group<64, 192, 2, 2>(ctx, a, g, 44); break;
  }
  if (rc) return rc;
  if (splits > 1) {
    hipLaunchKernelGGL(group_reduce, dim3((unsigned)cdiv(elems, 256)), dim3(256), 0, ctx->stream, g, a.Pp, elems, splits);
    GT_LAUNCHED(ctx);
  }
  return 0;
}
}

// C_i = dscale * D_i + pscale * A_i.B_i for a batch of `count` products (strides in elements; D laid out as C)
int gemm_scaled_batched(gt_ctx *ctx, int kind, int M, int N, int K, gt_buf A, int64_t sA, gt_buf B, int64_t sB, gt_buf D, int64_t sD,
                        float dscale, float pscale, gt_buf C, int64_t sC, int count) {
  return gemm_impl(ctx, kind, 0, M, N, K, A, sA, B, sB, C, sC, count, 0, 0, 0, D, sD, 1, dscale, pscale);
}

extern "C" {
int gt_gemm_sum(gt_ctx *ctx, int kind, int acc, int M, int N, int count, const int *K, const gt_buf *A, const gt_buf *B, gt_buf C) {
  GT_ENTER(ctx);
  GT_REQUIRE(ctx, count >= 1 && count <= 3 && K && A && B && C, "gt_gemm_sum: 1 to 3 products with their sizes and operands (got %d)", count);
  GT_REQUIRE(ctx, kind >= 0 && kind <= 2 && M >= 1 && N >= 1, "gt_gemm_sum: kind %d, M %d, N %d", kind, M, N);
  bool fused = count > 1 && kind != GT_TN && !ctx->opt_gemm_staged && C % 16 == 0 && N % 4 == 0 && (kind == GT_NT || N >= 4);
  for (int i = 0; i < count; i++) {
    GT_REQUIRE(ctx, K[i] >= 1 && A[i] && B[i], "gt_gemm_sum: product %d has K %d or a null operand", i, K[i]);
    fused = fused && K[i] % 32 == 0 && A[i] % 16 == 0 && B[i] % 16 == 0 && K[i] <= GT_DIRECT_LD_MAX;
  }
  fused = fused && N <= GT_DIRECT_LD_MAX;
  // the chained loop has one tile shape and no K split: below one workgroup per CU the single products, which pick
  // smaller tiles and split K, fill the chip better
  // Tile of the chained loop: 128 x 96, 128 x 160 or 128 x 128, whichever leaves the least idle in edge tiles and in the
  // last round of workgroups (two are resident per CU). 576 = 6 x 96; 640 = 4 x 160: a 16384-row output is 512 tiles, one
  // full round, where 128 x 128 makes 640 tiles for 512 slots and a quarter-full second round.
  int bn_sum = 128;
  {
    double best = 0;
    const int cands[3] = {128, 160, 96};
    for (int ci = 0; ci < 3; ci++) {
      const int bn = cands[ci];
      if (bn != 128 && N % bn != 0) continue;
      const double tiles = (double)cdiv(M, 128) * cdiv(N, bn), rounds = tiles / (2.0 * ctx->num_cu);
      const double score = ((double)M * N) / (tiles * 128.0 * bn) * (rounds / ceil(rounds));
      if (score > best * 1.02) { best = score; bn_sum = bn; }
    }
  }
  const bool t96 = bn_sum == 96, t160 = bn_sum == 160;
  if (fused && cdiv(M, 128) * cdiv(N, bn_sum) < (ctx->opt_gemm_sum_min_tiles >= 0 ? ctx->opt_gemm_sum_min_tiles : ctx->num_cu)) fused = false;
  if (!fused) {        // one launch per product, each adding to the one before
    for (int i = 0; i < count; i++)
      if (gemm_impl(ctx, kind, i ? 1 : acc, M, N, K[i], A[i], 0, B[i], 0, C, 0, 1)) return 1;
    return 0;
  }
  GemmArgs a;
  a.A = P<const float>(A[0]); a.B = P<const float>(B[0]); a.C = P<float>(C);
  a.M = M; a.N = N; a.K = K[0];
  a.lda = K[0]; a.ldb = kind == GT_NT ? K[0] : N; a.ldc = N;
  a.acc = acc; a.kchunk = K[0]; a.splits = 1; a.Pp = nullptr;
  a.sA = a.sB = a.sC = 0;
  a.zdiv = a.zgroup = 1; a.window = 0; a.sB2 = a.sC2 = 0;
  a.A2 = a.B2 = nullptr; a.K2 = 0; a.lda2 = a.ldb2 = 0;
  a.nx = count - 1; a.D = nullptr; a.sD = 0; a.scaled = 0; a.dscale = a.pscale = 1.f; a.rope = nullptr;
  double ksum = K[0];
  for (int i = 1; i < count; i++) {
    a.xA[i - 1] = P<const float>(A[i]); a.xB[i - 1] = P<const float>(B[i]);
    a.xK[i - 1] = K[i]; a.xlda[i - 1] = K[i]; a.xldb[i - 1] = kind == GT_NT ? K[i] : N;
    ksum += K[i];
  }
  char label[32];
  snprintf(label, sizeof label, "gemm.%s.128x%dx32", kind == GT_NT ? "nt" : "nn", bn_sum);
  ProfScope ps(ctx, label, 2.0 * M * N * ksum);
  if (kind == GT_NN)
    return t96 ? launch_multi<128, 96, 4, 1, GT_NN>(ctx, a, 30) : t160 ? launch_multi<128, 160, 4, 1, GT_NN>(ctx, a, 34)
                                                                       : launch_multi<128, 128, 2, 2, GT_NN>(ctx, a, 31);
  return t96 ? launch_multi<128, 96, 4, 1, GT_NT>(ctx, a, 32) : t160 ? launch_multi<128, 160, 4, 1, GT_NT>(ctx, a, 35)
                                                                     : launch_multi<128, 128, 2, 2, GT_NT>(ctx, a, 33);
}
int gt_gemm(gt_ctx *ctx, int kind, int acc, int M, int N, int K, gt_buf A, gt_buf B, gt_buf C) {
  return gemm_impl(ctx, kind, acc, M, N, K, A, 0, B, 0, C, 0, 1);
}
int gt_gemm_add(gt_ctx *ctx, int kind, int M, int N, int K, gt_buf A, gt_buf B, gt_buf D, gt_buf C) {
  if (ctx && !D) GT_FAIL(ctx, "gt_gemm_add: null addend");
  return gemm_impl(ctx, kind, 0, M, N, K, A, 0, B, 0, C, 0, 1, 0, 0, 0, D);
}
int gt_gemm_pair(gt_ctx *ctx, int kind, int acc, int M, int N, int K1, gt_buf A1, gt_buf B1, int K2, gt_buf A2, gt_buf B2,
                 gt_buf C) {
  if (ctx && (K2 < 1 || !A2 || !B2)) GT_FAIL(ctx, "gt_gemm_pair: the second product needs K2 >= 1 and both operands (got K2 = %d)", K2);
  // one K loop over both products for 16-byte aligned NT / NN operands; otherwise two launches, the second adding
  const int lda1 = kind == GT_TN ? M : K1, ldb1 = kind == GT_NT ? K1 : N, lda2 = kind == GT_TN ? M : K2, ldb2 = kind == GT_NT ? K2 : N;
  const bool fused = kind != GT_TN && K1 >= 1 && (lda1 % 4 == 0) && (ldb1 % 4 == 0) && (lda2 % 4 == 0) && (ldb2 % 4 == 0) &&
                     ((A1 | B1 | A2 | B2) % 16 == 0);
  if (fused) return gemm_impl(ctx, kind, acc, M, N, K1, A1, 0, B1, 0, C, 0, 1, K2, A2, B2);
  if (gemm_impl(ctx, kind, acc, M, N, K1, A1, 0, B1, 0, C, 0, 1)) return 1;
  return gemm_impl(ctx, kind, 1, M, N, K2, A2, 0, B2, 0, C, 0, 1);
}
int gt_gemm_batched(gt_ctx *ctx, int kind, int acc, int M, int N, int K, gt_buf A, int64_t strideA, gt_buf B,
                    int64_t strideB, gt_buf C, int64_t strideC, int count) {
  return gemm_impl(ctx, kind, acc, M, N, K, A, strideA, B, strideB, C, strideC, count);
}
}
