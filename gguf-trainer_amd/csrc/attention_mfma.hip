// Attention forward / backward on the FP32 matrix cores (v_mfma_f32_32x32x2_f32). This file is compiled once per
// supported head dim (-DHD=32, -DHD=64, -DHD=128); the entry points carry the head dim in their names.
// Same math and saved statistic as the generic kernels in attention.hip: causal / sliding window,
// GQA, scores in the log2 domain, softmax recomputed in backward from lse2.
//
// How the tiles map onto a 64-lane wavefront. A wavefront owns 32 queries (forward, dQ) or 32 keys
// (dK/dV); a workgroup is four of them. Scores are computed TRANSPOSED, S^T[key][query] = K.Q^T
// (forward, dQ), so that an accumulator lane holds ONE query (column lane%32) and 16 keys: the
// softmax row statistics are per-lane scalars and the row reduction is in-register plus one
// cross-half shuffle. In dK/dV it is S[query][key] = Q.K^T, one key per lane. Either way the 16
// accumulator registers of a lane sit at rows 8*(r/4) + 4*(lane/32) + r%4, which is exactly the K
// index order an MFMA step sequence consumes when step i takes row 8*(i/4) + 4*(lane/32) + i%4 from
// its half: the probability / dS tile feeds the second contraction (P.V, dS.K, P^T.dO, dS^T.Q)
// straight from the accumulators, with no transpose through LDS.
//
// Operand staging. The tile that changes per iteration (K,V in forward and dQ; Q,dO in dK/dV) is
// staged in LDS in the layout its contraction reads with ds_read_b128, one read per four MFMAs:
// row-major [row][hd+4] for the first contraction (a lane's four consecutive head dims of its row)
// and transposed [hd][rows+4] for the second (a lane's four consecutive rows of its head dim).
// Strides of 4 mod 32 words keep every 8-lane group of a b128 access on distinct banks, and the
// global->LDS copy assigns consecutive lanes to consecutive rows so both stores are conflict-free.
// The operand that stays fixed for the whole loop (this lane's query / key row) lives in registers.
// Forward and dK/dV keep two LDS buffers for the changing tile: while a stage computes on one, the next stage's
// tile is written to the other from the registers its global loads filled earlier, and one barrier ends the
// stage. Those loads take rows past the end of a sequence from its last row instead of testing bounds, so a
// stage has no branch between its MFMAs and the scheduler can lay the loads, LDS stores and softmax arithmetic
// under them. All LDS reads of a contraction are issued before its first MFMA.
//
// The running maximum of the online softmax is only raised, and the output accumulators rescaled,
// when some lane of the wavefront actually sees a larger score (after the first few tiles it almost
// never does), which keeps the accumulators out of the VALU in the steady state.
//
// dK/dV loops over the query heads of the kv group inside the workgroup and over query tiles in
// increasing order, so the GQA sum has a fixed order and needs no atomics.
//
// Kept scores. With a scores buffer (T a multiple of 128) the forward stores its scores, one [key][query] 32 x 32
// block per (key sub-tile, query stage) of every (sequence, head), and dK/dV reads them back instead of recomputing
// Q.K^T: three contractions per stage there instead of four.
//
// Kept score gradients. With a dS workspace (T a multiple of 128) dK/dV stores the score
// gradients it computes, and dQ = dS.K is one banded batched product afterwards (gemm.hip) instead of a kernel that
// recomputes S and dP: one [T][T] matrix per (sequence, head), kept in blocks [row tile of 128][key step of 32]
// [128 rows][32 keys], in which every block inside a row tile's band of keys is written (zeros where no pair is live).
//
// Small launches (one short sequence, few heads) have fewer tiles than the chip has CUs and their time is the
// serial loop of the longest tile. For them p.splits > 1 cuts every tile's loop range (key stages in forward and
// dQ, query stages in dK/dV) into that many workgroups, which write partial results (unnormalised output with
// its running maximum and sum; partial dQ; dK/dV slices) that a second kernel folds in split order.
#include <algorithm>
#include <type_traits>
#include "common.h"
#include "bf16_pieces.h"

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

struct AttnP {
  int B, T, Hq, Hkv, hd, window;
  float c2;
  float scale;
  int splits;               // >= 1: the loop range of every tile is cut into this many workgroups (small launches)
};

#ifndef HD
#error "compile with -DHD=32, -DHD=64 or -DHD=128"
#endif
#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, HD)
#define NEG_BIG (-1.0e30f)
#define LD (HD + 4)          // row-major tile stride

namespace {                  // per-head-dim helpers: each translation unit has its own

__device__ __forceinline__ int win_lo_m(int t, int window) { return (window > 0 && t + 1 > window) ? t + 1 - window : 0; }
__device__ __forceinline__ int acc_row(int r, int g) { return 8 * (r / 4) + 4 * g + (r % 4); }
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ROWS x HD tile. Global loads are coalesced (16 lanes cover one 256-byte row). Row-major copy:
// [row][LD]. Transposed copy: [d][ROWS+4] with the 16-byte column chunks XOR-swizzled by (d/8)%8, which
// makes the scalar transposing stores hit every bank exactly twice per 64 lanes (the minimum) while the
// b128 reads of the second contraction stay conflict-free (an aligned group of 8 lanes shares d/8).
template <int ROWS> struct TileIO {
  static constexpr int LDT = ROWS + 4;
  static constexpr int PER = (ROWS * HD / 4) / 256;
  // Where this thread's float4 units sit inside a tile whose first row is at `base`: computed once per kernel. A stage's
  // loads are then `base + off[i]` with a wave-uniform base that advances from stage to stage (scalar arithmetic) and a
  // 32-bit lane offset. A row past the end of the matrix (the last tile, when fewer than ROWS rows are left: nvalid < ROWS)
  // reads the matrix's last row instead: no bounds test and no branch, so the loads can be scheduled among the MFMAs around
  // them. What such a row holds is finite and every product it enters is masked to zero by the kernels (a query or key
  // past the end is never live), so the results are those of a zero-filled tile.
  __device__ static __forceinline__ void offsets(unsigned (&off)[PER], size_t stride, int tid) {      // in bytes
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int u = tid + i * 256, row = u / (HD / 4), c4 = u % (HD / 4);
      off[i] = (unsigned)((row * stride + c4 * 4) * sizeof(float));
    }
  }
  __device__ static __forceinline__ void load(v4f (&reg)[PER], const float *__restrict__ base, const unsigned (&off)[PER], unsigned stride,
                                              int nvalid, int tid) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int row = (tid + i * 256) / (HD / 4);
      unsigned back = (unsigned)max(row - (nvalid - 1), 0) * (stride * (unsigned)sizeof(float));      // 0 inside the matrix
      reg[i] = *reinterpret_cast<const v4f *>(reinterpret_cast<const char *>(base) + (off[i] - back));   // uniform base + 32-bit lane offset
    }
  }
  __device__ static __forceinline__ void store_rows(const v4f (&reg)[PER], float *lds, int tid) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int u = tid + i * 256, row = u / (HD / 4), c4 = u % (HD / 4);
      *reinterpret_cast<v4f *>(lds + row * LD + c4 * 4) = reg[i];
    }
  }
  __device__ static __forceinline__ void store_t(const v4f (&reg)[PER], float *ldst, int tid) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      int u = tid + i * 256, row = u / (HD / 4), c4 = u % (HD / 4);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        int d = c4 * 4 + j;
        ldst[d * LDT + 4 * ((row >> 2) ^ ((d >> 3) & 7)) + (row & 3)] = reg[i][j];
      }
    }
  }
};

// this lane's row as MFMA B-operand registers: reg[4j+s] = x[8j + 4g + s] * mul
__device__ __forceinline__ void load_row_regs(float (&reg)[HD / 2], const float *__restrict__ row, bool valid, int g, float mul) {
#pragma unroll
  for (int j = 0; j < HD / 8; j++) {
    v4f v = {0.f, 0.f, 0.f, 0.f};
    if (valid) v = *reinterpret_cast<const v4f *>(row + 8 * j + 4 * g);
#pragma unroll
    for (int s = 0; s < 4; s++) reg[4 * j + s] = v[s] * mul;
  }
}

// acc = Tile(32 rows starting at `rows`) . reg^T : A = rows of the row-major tile, B = this lane's registers.
// The LDS reads are issued eight b128 at a time, ahead of the MFMAs that consume them.
template <int NBMAX = 8>
__device__ __forceinline__ v16f rows_dot_regs(const float *rows, const float (&reg)[HD / 2], int l32, int g) {
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  constexpr int NB = HD / 8 < NBMAX ? HD / 8 : NBMAX;       // b128 reads in flight per batch
#pragma unroll
  for (int j0 = 0; j0 < HD / 8; j0 += NB) {
    v4f a[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) a[j] = *reinterpret_cast<const v4f *>(rows + l32 * LD + 8 * (j0 + j) + 4 * g);
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
      for (int s = 0; s < 4; s++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j][s], reg[4 * (j0 + j) + s], acc, 0, 0, 0);
  }
  return acc;
}

// out[dt] += TileT(cols [col0, col0+32)) . w : A = the transposed tile (stride LDT), B = 16 accumulator-ordered weights
template <int LDT, int INFLIGHT = 8>
__device__ __forceinline__ void t_dot_acc(v16f (&out)[HD / 32], const float *ldst, int col0, const float (&w)[16], int l32, int g) {
  constexpr int DT = HD / 32;
  constexpr int QB = INFLIGHT / DT >= 4 ? 4 : (INFLIGHT / DT >= 2 ? 2 : 1);    // column chunks fetched ahead: INFLIGHT b128 reads in flight
#pragma unroll
  for (int q0 = 0; q0 < 4; q0 += QB) {
    v4f a[DT][QB];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int q = 0; q < QB; q++) {
        int d = dt * 32 + l32, chunk = (col0 >> 2) + 2 * (q0 + q) + g;
        a[dt][q] = *reinterpret_cast<const v4f *>(ldst + d * LDT + 4 * (chunk ^ ((d >> 3) & 7)));
      }
#pragma unroll
    for (int q = 0; q < QB; q++)
#pragma unroll
      for (int s = 0; s < 4; s++)
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
          out[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[dt][q][s], w[4 * (q0 + q) + s], out[dt], 0, 0, 0);
  }
}

// ---- attention's contractions on the bf16 matrix instruction (bf16_pieces.h): a lane's 8 consecutive k per MFMA --------------------------
// this lane's row as pieces: qp[c] = pieces of x[16c + 8g + (0..7)] * mul
__device__ __forceinline__ void load_row_pieces(v4u (&qp)[HD / 16][3], const float *__restrict__ row, bool valid, int g, float mul) {
#pragma unroll
  for (int c = 0; c < HD / 16; c++) {
    v4f lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
    if (valid) { lo = *reinterpret_cast<const v4f *>(row + 16 * c + 8 * g); hi = *reinterpret_cast<const v4f *>(row + 16 * c + 8 * g + 4); }
    const float x[8] = {lo[0] * mul, lo[1] * mul, lo[2] * mul, lo[3] * mul, hi[0] * mul, hi[1] * mul, hi[2] * mul, hi[3] * mul};
    cut8(x, qp[c]);
  }
}
// acc[n] = Tile(32 rows starting at rows + n * 32 * LD) . row^T for N sub-tiles at once: their MFMAs alternate, so that (for N > 1) no MFMA
// waits for the one before it on the same accumulator
template <int N>
__device__ __forceinline__ void rows_dot_pieces(v16f (&acc)[N], const float *rows, const v4u (&qp)[HD / 16][3], int l32, int g) {
  constexpr int TA[6] = GT_PIECE_TERMS_A, TB[6] = GT_PIECE_TERMS_B;
#pragma unroll
  for (int n = 0; n < N; n++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[n][r] = 0.f;
  if constexpr (N == 1 && HD >= 128) {          // one sub-tile, registers to spare: its six terms alternate between two accumulators
    v16f other;
#pragma unroll
    for (int r = 0; r < 16; r++) other[r] = 0.f;
#pragma unroll
    for (int c = 0; c < HD / 16; c++) {
      v4u ka[3];
      const float *src = rows + l32 * LD + 16 * c + 8 * g;
      const v4f lo = *reinterpret_cast<const v4f *>(src), hi = *reinterpret_cast<const v4f *>(src + 4);
      const float x[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      cut8(x, ka);
#pragma unroll
      for (int t = 0; t < 6; t += 2) {
        other = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, ka[TA[t]]), __builtin_bit_cast(v8bf, qp[c][TB[t]]), other, 0, 0, 0);
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, ka[TA[t + 1]]), __builtin_bit_cast(v8bf, qp[c][TB[t + 1]]), acc[0], 0, 0, 0);
      }
    }
    acc[0] += other;
    return;
  }
#pragma unroll
  for (int c = 0; c < HD / 16; c++) {
    v4u ka[N][3];
#pragma unroll
    for (int n = 0; n < N; n++) {
      const float *src = rows + (n * 32 + l32) * LD + 16 * c + 8 * g;
      const v4f lo = *reinterpret_cast<const v4f *>(src), hi = *reinterpret_cast<const v4f *>(src + 4);
      const float x[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      cut8(x, ka[n]);
    }
#pragma unroll
    for (int t = 0; t < 6; t++)
#pragma unroll
      for (int n = 0; n < N; n++)
        acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, ka[n][TA[t]]), __builtin_bit_cast(v8bf, qp[c][TB[t]]), acc[n], 0, 0, 0);
  }
}
// out[dt] += TileT(cols [col0, col0+32)) . w, w in accumulator order: MFMA j takes w[8j .. 8j+7], the keys 16j + 4g + (0..3) and 16j + 8 + 4g + (0..3)
template <int LDT>
__device__ __forceinline__ void t_dot_pieces(v16f (&out)[HD / 32], const float *ldst, int col0, const float (&w)[16], int l32, int g) {
  constexpr int DT = HD / 32;
  constexpr int TA[6] = GT_PIECE_TERMS_A, TB[6] = GT_PIECE_TERMS_B;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    v4u pw[3], va[DT][3];
    const float xw[8] = {w[8 * j], w[8 * j + 1], w[8 * j + 2], w[8 * j + 3], w[8 * j + 4], w[8 * j + 5], w[8 * j + 6], w[8 * j + 7]};
    cut8(xw, pw);
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      const int d = dt * 32 + l32, chunk = (col0 >> 2) + 4 * j + g;
      const v4f lo = *reinterpret_cast<const v4f *>(ldst + d * LDT + 4 * (chunk ^ ((d >> 3) & 7)));
      const v4f hi = *reinterpret_cast<const v4f *>(ldst + d * LDT + 4 * ((chunk + 2) ^ ((d >> 3) & 7)));
      const float x[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      cut8(x, va[dt]);
    }
#pragma unroll
    for (int t = 0; t < 6; t++)
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
        out[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, va[dt][TA[t]]), __builtin_bit_cast(v8bf, pw[TB[t]]), out[dt], 0, 0, 0);
  }
}

// ---- dK/dV on pieces: the query-side tiles cut ONCE per workgroup, as they are stored, into planes of bf16 pairs ----
// A thread stores columns d = 4 (tid % 8) + (0..3) and d + 32 of row tid / 8 of a 32 x 64 tile; cutting (row, d) and (row, d + 32)
// together gives one word per piece (h, m or l): the low and the high half. Row-major planes [piece][row][32 words] keep those words:
// they feed the contraction over the head dim, whose k-slots then run d, d + 32, d + 1, d + 33, ... (the other operand, this lane's own
// row, is cut in the same order). Transposed planes [piece][d = 0..63][16 words] feed the contractions over the rows and hold two ROWS
// of one column to a word (see pl_store_t). In both, 16-byte chunks of a plane row are XOR-swizzled so that the b128 reads of 8
// consecutive lanes cover all banks.
#define PL_PLANE 1024                                   // words per plane
#define PL_GR 0                                          // dO, row-major
#define PL_GT (3 * PL_PLANE)                             // dO, transposed
#define PL_QT (6 * PL_PLANE)                             // Q, transposed
#define PL_L (9 * PL_PLANE)                              // lse, then D
#define PL_BUF (9 * PL_PLANE + 2 * 32)                   // words per buffer
// this thread's share of a tile: row tid / 8, columns 4 (tid % 8) + (0..3) in x0 and 32 more in x1, cut into words w[piece][e]
__device__ __forceinline__ void pl_cut_unit(const v4f &x0, const v4f &x1, unsigned (&w)[3][4]) {
#pragma unroll
  for (int e = 0; e < 4; e++) split_pair(x0[e], x1[e], w[0][e], w[1][e], w[2][e]);
}
__device__ __forceinline__ void pl_store_rows(const unsigned (&w)[3][4], unsigned *planes, int tid) {
  const int row = tid / 8, c = tid % 8;
#pragma unroll
  for (int pc = 0; pc < 3; pc++)
    *reinterpret_cast<v4u *>(planes + pc * PL_PLANE + row * 32 + 4 * (c ^ (row & 7))) = v4u{w[pc][0], w[pc][1], w[pc][2], w[pc][3]};
}
// transposed planes: word (d, pair of rows) = the pieces of (row, d) and (row + 1, d), row even. The thread of the even row and the
// thread of the odd row (8 lanes apart in a DPP row) exchange their words; the even one then writes the word of column d, the odd
// one that of column d + 32. Words of a 64-byte plane row are ordered so that the 8 k-slots of a lane are one 16-byte chunk; chunks are
// XOR-swizzled within a row (reads conflict-free; a wavefront's stores, 8 columns 4 apart of 8 rows, meet four by four: telling them apart
// by one more address bit costs the two registers the kernel does not have).
__device__ __forceinline__ int pl_swz_t(int d) { return ((d >> 1) & 3) ^ ((d >> 3) & 3); }
__device__ __forceinline__ void pl_store_t(const unsigned (&w)[3][4], unsigned *planes, int tid) {
  const int row = tid / 8, c = tid % 8, odd = row & 1, pr = row >> 1;
  const unsigned sel = odd ? 0x03020706u : 0x05040100u;
  const int pos = (pr & 9) | ((pr & 4) >> 1) | ((pr & 2) << 1);          // pair 8j + 4i + 2g + s sits at word 8j + 4g + 2i + s
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const int d = 32 * odd + 4 * c + e, at = d * 16 + 4 * ((pos >> 2) ^ pl_swz_t(d)) + (pos & 3);
#pragma unroll
    for (int pc = 0; pc < 3; pc++) {
      const unsigned other = (unsigned)__builtin_amdgcn_mov_dpp((int)w[pc][e], 0x128, 0xf, 0xf, true);          // row_ror:8: the partner's word
      planes[pc * PL_PLANE + at] = __builtin_amdgcn_perm(other, w[pc][e], sel);
    }
  }
}
// this lane's row in the planes' k-slot order: vp[c][piece] word e = pieces of (x[8c + 4g + e], x[32 + 8c + 4g + e]) * mul
__device__ __forceinline__ void pl_load_row(v4u (&vp)[4][3], const float *__restrict__ row, bool valid, int g, float mul) {
#pragma unroll
  for (int c = 0; c < 4; c++) {
    v4f lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
    if (valid) { lo = *reinterpret_cast<const v4f *>(row + 8 * c + 4 * g); hi = *reinterpret_cast<const v4f *>(row + 32 + 8 * c + 4 * g); }
#pragma unroll
    for (int e = 0; e < 4; e++) {
      unsigned h, m, l;
      split_pair(lo[e] * mul, hi[e] * mul, h, m, l);
      vp[c][0][e] = h; vp[c][1][e] = m; vp[c][2][e] = l;
    }
  }
}
// Tile(32 rows, row-major planes) . row^T: four steps of 16 k-slots, six piece products each, no vector work at all
__device__ __forceinline__ v16f pl_rows_dot(const unsigned *planes, const v4u (&vp)[4][3], int l32, int g) {
  constexpr int TA[6] = GT_PIECE_TERMS_A, TB[6] = GT_PIECE_TERMS_B;
  v16f acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  v4u a[2][3];
  auto fetch = [&](int c) {
#pragma unroll
    for (int pc = 0; pc < 3; pc++) a[c & 1][pc] = *reinterpret_cast<const v4u *>(planes + pc * PL_PLANE + l32 * 32 + 4 * ((2 * c + g) ^ (l32 & 7)));
  };
  fetch(0);
#pragma unroll
  for (int c = 0; c < 4; c++) {          // the next step's operand is asked for before this step's MFMAs, and no further ahead
    if (c < 3) fetch(c + 1);
#pragma unroll
    for (int t = 0; t < 6; t++)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a[c & 1][TA[t]]), __builtin_bit_cast(v8bf, vp[c][TB[t]]), acc, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
  return acc;
}
// out[dt] += TileT(transposed planes) . w, w in accumulator order (MFMA j takes w[8j .. 8j+7]: rows 16j + 4g + (0..3) and 16j + 8 + 4g + (0..3))
__device__ __forceinline__ void pl_t_dot(v16f (&out)[HD / 32], const unsigned *planes, const float (&w)[16], int l32, int g) {
  constexpr int TA[6] = GT_PIECE_TERMS_A, TB[6] = GT_PIECE_TERMS_B;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    v4u pw[3];
    const float xw[8] = {w[8 * j], w[8 * j + 1], w[8 * j + 2], w[8 * j + 3], w[8 * j + 4], w[8 * j + 5], w[8 * j + 6], w[8 * j + 7]};
    cut8(xw, pw);
    v4u va[HD / 32][3];
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
      for (int pc = 0; pc < 3; pc++) {
        const int d = 32 * dt + l32;
        va[dt][pc] = *reinterpret_cast<const v4u *>(planes + pc * PL_PLANE + d * 16 + 4 * ((2 * j + g) ^ pl_swz_t(d)));
      }
#pragma unroll
    for (int t = 0; t < 6; t++)          // the blocks' chains alternate
#pragma unroll
      for (int dt = 0; dt < HD / 32; dt++)
        out[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, va[dt][TA[t]]), __builtin_bit_cast(v8bf, pw[TB[t]]), out[dt], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
}

__device__ __forceinline__ void store_row(float *row, const v16f (&acc)[HD / 32], int g, float mul, int add) {
  v4f old[HD / 32][4];
  if (add) {          // every old value first: a load behind a store to the same array would wait for it
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
      for (int a = 0; a < 4; a++) old[dt][a] = *reinterpret_cast<const v4f *>(row + dt * 32 + 8 * a + 4 * g);
  }
#pragma unroll
  for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
    for (int a = 0; a < 4; a++) {
      v4f o = {acc[dt][4 * a] * mul, acc[dt][4 * a + 1] * mul, acc[dt][4 * a + 2] * mul, acc[dt][4 * a + 3] * mul};
      if (add) o += old[dt][a];
      *reinterpret_cast<v4f *>(row + dt * 32 + 8 * a + 4 * g) = o;
    }
}

// store_row for a gradient with respect to ROTATED rows (q or k after rope) whose caller wants the gradient with respect
// to the rows before the rotation: (lo, hi) = (c lo + s hi, -s lo + c hi) per pair (j, j + HD/2), srcRope's backward
// (wgsl.ts:346-384), applied to the accumulators on their way out. A lane holds whole rows, so both halves of every pair
// are its own registers. cs: this row's (cos, sin) pairs, HD floats. Two float4 units of the low half at a time.
__device__ __forceinline__ void store_row_rot(float *row, const v16f (&acc)[HD / 32], int g, float mul, int add, const float *__restrict__ cs) {
  constexpr int NU = HD / 16;                    // float4 units in the low half of a row
#pragma unroll
  for (int u0 = 0; u0 < NU; u0 += 2) {
    v4f lo[2], hi[2], c0[2], c1[2], olo[2], ohi[2];
    int col[2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
      const int u = u0 + q;
      const int dt = HD >= 64 ? u / 4 : 0, a = HD >= 64 ? u % 4 : u;
      const int dth = HD >= 64 ? dt + HD / 64 : 0, ah = HD >= 64 ? a : a + 2;
      col[q] = dt * 32 + 8 * a + 4 * g;
      lo[q] = v4f{acc[dt][4 * a], acc[dt][4 * a + 1], acc[dt][4 * a + 2], acc[dt][4 * a + 3]} * mul;
      hi[q] = v4f{acc[dth][4 * ah], acc[dth][4 * ah + 1], acc[dth][4 * ah + 2], acc[dth][4 * ah + 3]} * mul;
      c0[q] = *reinterpret_cast<const v4f *>(cs + 2 * col[q]);
      c1[q] = *reinterpret_cast<const v4f *>(cs + 2 * col[q] + 4);
      if (add) {
        olo[q] = *reinterpret_cast<const v4f *>(row + col[q]);
        ohi[q] = *reinterpret_cast<const v4f *>(row + col[q] + HD / 2);
      }
    }
#pragma unroll
    for (int q = 0; q < 2; q++) {
      const v4f c = {c0[q][0], c0[q][2], c1[q][0], c1[q][2]}, sn = {c0[q][1], c0[q][3], c1[q][1], c1[q][3]};
      v4f r0 = c * lo[q] + sn * hi[q], r1 = -sn * lo[q] + c * hi[q];
      if (add) { r0 += olo[q]; r1 += ohi[q]; }
      *reinterpret_cast<v4f *>(row + col[q]) = r0;
      *reinterpret_cast<v4f *>(row + col[q] + HD / 2) = r1;
    }
  }
}
// rot: the rotation table ([T][HD/2] (cos, sin) pairs) when the destination wants the gradient before the rotation, else null
__device__ __forceinline__ void store_grad_row(float *row, const v16f (&acc)[HD / 32], int g, float mul, int add, const float *rot, int t) {
  if (rot) store_row_rot(row, acc, g, mul, add, rot + (size_t)t * HD);
  else store_row(row, acc, g, mul, add);
}

}  // namespace

#define KT (HD <= 64 ? 64 : 32)      // keys per LDS stage in forward and dQ
// forward and dK/dV are held to the registers of two wavefronts per SIMD up to head dim 64 (two workgroups per CU); at 128 one
#define WAVES_PER_SIMD (HD <= 64 ? 2 : 1)
#define NSUB (KT / 32)

// ---- forward --------------------------------------------------------------------------------------
// KEEP: the scores are stored for dK/dV (sco).
// The K and V^T tiles are double-buffered in LDS: the tile of stage kt+1 is written (from the registers its global loads
// filled during stage kt-1) while stage kt computes on the other buffer, the loads of stage kt+2 follow, and one barrier
// ends the stage. A stage in which every 32-key sub-tile has a visible pair for this wavefront (all but the stages at the
// diagonal and at a window's edge) is straight-line code, masks applied by one unsigned compare per element, so that the
// scheduler can run the softmax of one sub-tile, the LDS stores and the loads under the MFMAs of another.
#define FWD_BUF (KT * LD + HD * (KT + 4))        // floats per buffer: K rows, V transposed
#define FWD_SMEM (2 * FWD_BUF * sizeof(float))
// PX: both contractions on the bf16 matrix instruction (the query row, the K and V^T tiles and the probabilities as bf16 pieces, cut in
// registers by every wavefront that reads them).
template <bool KEEP, bool PX = false>
__global__ __launch_bounds__(256, WAVES_PER_SIMD) void FN(attn_fwd_mfma_k)(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                       const float *__restrict__ v, float *__restrict__ out,
                                                       float *__restrict__ lse, float *__restrict__ fpart, float *sco) {
  using IO = TileIO<KT>;
  constexpr int FWD_NB = 8;          // LDS reads in flight per contraction
  extern __shared__ __attribute__((aligned(16))) float fwd_smem[];      // 2 x 35 KB at hd 64 and 128
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, g = lane / 32, l32 = lane % 32;
  // 1-D grid ordered by work: every (head, sequence) pair's longest query tile is dispatched before any shorter
  // one, so the causal triangle packs onto the CUs without a long tail
  const int nhb = p.Hq * p.B;
  const int sp = (int)(blockIdx.x % p.splits);
  const unsigned bid = blockIdx.x / p.splits;
  const int qtile = (int)((p.T + 127) / 128) - 1 - (int)(bid / nhb);
  const int h = (bid % nhb) % p.Hq, b = (bid % nhb) / p.Hq;
  const int kvh = h / (p.Hq / p.Hkv);
  const size_t qstr = (size_t)p.Hq * HD, kstr = (size_t)p.Hkv * HD;
  const int tq0 = qtile * 128 + wave * 32, t = tq0 + l32;
  const int tq1 = min(tq0 + 31, p.T - 1);
  const bool tv = t < p.T;
  const float *kb = k + (size_t)b * p.T * kstr + (size_t)kvh * HD;
  const float *vb = v + (size_t)b * p.T * kstr + (size_t)kvh * HD;
  float qreg[PX ? 1 : HD / 2];
  v4u qp[PX ? HD / 16 : 1][3];
  if constexpr (PX) load_row_pieces(qp, q + ((size_t)b * p.T + (tv ? t : 0)) * qstr + (size_t)h * HD, tv, g, p.c2);
  else load_row_regs(qreg, q + ((size_t)b * p.T + (tv ? t : 0)) * qstr + (size_t)h * HD, tv, g, p.c2);
  // the two contractions of a 32-key sub-tile, either way
  auto scores1 = [&](const float *rows) {
    if constexpr (PX) { v16f a1[1]; rows_dot_pieces<1>(a1, rows, qp, l32, g); return a1[0]; }
    else return rows_dot_regs<FWD_NB>(rows, qreg, l32, g);
  };
  auto weighted = [&](v16f (&o)[HD / 32], const float *ldst, int col0, const float (&w)[16]) {
    if constexpr (PX) t_dot_pieces<IO::LDT>(o, ldst, col0, w, l32, g);
    else t_dot_acc<IO::LDT, FWD_NB>(o, ldst, col0, w, l32, g);
  };
  const int lo_t = win_lo_m(t, p.window);
  int kt_lo = win_lo_m(qtile * 128, p.window) / KT;
  int kt_hi = min(p.T - 1, qtile * 128 + 127) / KT;
  if (p.splits > 1) {                      // this workgroup's share of the key stages (possibly none)
    const int n = kt_hi - kt_lo + 1, first = kt_lo;
    kt_lo = first + sp * n / p.splits;
    kt_hi = first + (sp + 1) * n / p.splits - 1;
  }
  const int wave_lo = win_lo_m(tq0, p.window), wave_lo_last = win_lo_m(tq1, p.window);
  const bool ragged = tq0 + 31 >= p.T;

  v16f oacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[dt][r] = 0.f;
  float m = NEG_BIG, l = 0.f;

  // One set of staging registers serves both tiles: the K tile of the next stage is loaded at the top of a stage and
  // written to the idle buffer in its middle, the V tile is loaded there and written at the stage's end. A stage index past
  // the last one is clamped to it (its tiles are loaded, and written to the idle buffer, once more, which nobody reads):
  // the loop body has no test for "is there a next stage".
  v4f pt[IO::PER];
  unsigned koffs[IO::PER];
  IO::offsets(koffs, kstr, tid);
  auto load_tile = [&](const float *base, int kt) {
    kt = min(kt, kt_hi);
    IO::load(pt, base + (size_t)kt * KT * kstr, koffs, (unsigned)kstr, KEEP ? KT : p.T - kt * KT, tid);      // (kept scores: T is a multiple of 128, no tile is short: no clamp arithmetic; 3 % at head dim 128)
  };
  if (kt_lo <= kt_hi) {
    load_tile(kb, kt_lo);
    IO::store_rows(pt, fwd_smem, tid);
    load_tile(vb, kt_lo);
    IO::store_t(pt, fwd_smem + KT * LD, tid);
    __syncthreads();
  }
  for (int kt = kt_lo; kt <= kt_hi; kt++) {
    const float *sK = fwd_smem + ((kt - kt_lo) & 1) * FWD_BUF, *sVt = sK + KT * LD;
    float *nxt = fwd_smem + (((kt - kt_lo) & 1) ^ 1) * FWD_BUF;
    load_tile(kb, kt + 1);
    bool act[NSUB];
    bool plain = tq0 < p.T, any_act = false;      // plain: every pair of every sub-tile is visible to this wavefront
#pragma unroll
    for (int sub = 0; sub < NSUB; sub++) {
      const int k0 = kt * KT + sub * 32;
      act[sub] = tq0 < p.T && !(k0 > tq1 || k0 + 31 < wave_lo);           // wave-uniform: some (query, key) pair is visible
      plain = plain && !(ragged || k0 + 31 > tq0 || k0 < wave_lo_last);
      any_act = any_act || act[sub];
    }
    // where the scores (log2 domain; -1e30 where masked, which dK/dV masks again) of a 32 x 32 block go for dK/dV: [key][query], 4 KB in one piece
    float *sb = KEEP ? sco + ((((size_t)b * p.Hq + h) * (unsigned)(p.T / 32) + (unsigned)(kt * KT) / 32) * (unsigned)(p.T / 32) + (unsigned)tq0 / 32) * 1024 + l32
                     : nullptr;
    float pr[NSUB][16];
    if (plain) {
      float mx = NEG_BIG;
      v16f sall[NSUB];
      if constexpr (PX) rows_dot_pieces<NSUB>(sall, sK, qp, l32, g);
#pragma unroll
      for (int sub = 0; sub < NSUB; sub++) {
        v16f s;
        if constexpr (PX) s = sall[sub];
        else s = rows_dot_regs<FWD_NB>(sK + sub * 32 * LD, qreg, l32, g);
#pragma unroll
        for (int r = 0; r < 16; r++) {
          pr[sub][r] = s[r];
          mx = fmaxf(mx, s[r]);
        }
        if (KEEP) {
#pragma unroll
          for (int r = 0; r < 16; r++)                // read again only in the backward
            __builtin_nontemporal_store(pr[sub][r], sb + (size_t)sub * (p.T / 32) * 1024 + acc_row(r, g) * 32);
        }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      if (__any(mx > m)) {                                      // rare after the first tiles
        const float mn = fmaxf(m, mx);
        const float alpha = fast_exp2(m - mn);
        l *= alpha;
        m = mn;
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
          for (int r = 0; r < 16; r++) oacc[dt][r] *= alpha;
      }
#pragma unroll
      for (int sub = 0; sub < NSUB; sub++) {
        float ls = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          float e = fast_exp2(pr[sub][r] - m);          // every score is a number and m is at least their maximum
          pr[sub][r] = e;
          ls += e;
        }
        l += ls;
        if (sub == 0) {           // independent of the MFMAs around them
          IO::store_rows(pt, nxt, tid);
          load_tile(vb, kt + 1);
        }
        weighted(oacc, sVt, sub * 32, pr[sub]);
      }
    } else {
      IO::store_rows(pt, nxt, tid);
      load_tile(vb, kt + 1);
      if (any_act) {
        bool msk[NSUB];
        float mx = NEG_BIG;
#pragma unroll
        for (int sub = 0; sub < NSUB; sub++) {
          if (!act[sub]) continue;
          const int k0 = kt * KT + sub * 32;
          v16f s = scores1(sK + sub * 32 * LD);
          const bool need_mask = ragged || k0 + 31 > tq0 || k0 < wave_lo_last;
          msk[sub] = need_mask;
          if (need_mask) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
              int key = k0 + acc_row(r, g);
              pr[sub][r] = (tv && key <= t && key >= lo_t) ? s[r] : NEG_BIG;
            }
          } else {
#pragma unroll
            for (int r = 0; r < 16; r++) pr[sub][r] = s[r];
          }
#pragma unroll
          for (int r = 0; r < 16; r++) mx = fmaxf(mx, pr[sub][r]);
          if (KEEP) {
#pragma unroll
            for (int r = 0; r < 16; r++) __builtin_nontemporal_store(pr[sub][r], sb + (size_t)sub * (p.T / 32) * 1024 + acc_row(r, g) * 32);
          }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        if (__any(mx > m)) {
          const float mn = fmaxf(m, mx);
          const float alpha = fast_exp2(m - mn);
          l *= alpha;
          m = mn;
#pragma unroll
          for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[dt][r] *= alpha;
        }
#pragma unroll
        for (int sub = 0; sub < NSUB; sub++) {
          if (!act[sub]) continue;
          float ls = 0.f;
#pragma unroll
          for (int r = 0; r < 16; r++) {
            // a masked score is NEG_BIG; with m still NEG_BIG (no visible key yet) the difference would be 0
            float e = (!msk[sub] || pr[sub][r] > -1.0e29f) ? fast_exp2(pr[sub][r] - m) : 0.f;
            pr[sub][r] = e;
            ls += e;
          }
          l += ls;
          weighted(oacc, sVt, sub * 32, pr[sub]);
        }
      }
    }
    IO::store_t(pt, nxt + KT * LD, tid);
    __syncthreads();
  }
  const float lt = l + __shfl_xor(l, 32, 64);
  if (!tv) return;
  const size_t sidx = ((size_t)b * p.Hq + h) * p.T + t;
  if (p.splits > 1) {        // partial: unnormalised output, running maximum and sum of this key range
    const size_t slice = (size_t)p.B * p.T * qstr, rows = (size_t)p.B * p.Hq * p.T;
    store_row(fpart + sp * slice + ((size_t)b * p.T + t) * qstr + (size_t)h * HD, oacc, g, 1.0f, 0);
    if (g == 0) {
      float *mp = fpart + (size_t)p.splits * slice;
      mp[sp * rows + sidx] = m;
      mp[((size_t)p.splits + sp) * rows + sidx] = lt;
    }
    return;
  }
  store_row(out + ((size_t)b * p.T + t) * qstr + (size_t)h * HD, oacc, g, 1.0f / lt, 0);
  if (g == 0) lse[sidx] = m + log2f(lt);
}

// ---- dQ -----------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void FN(attn_bwd_dq_mfma_k)(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                          const float *__restrict__ v, const float *__restrict__ go,
                                                          const float *__restrict__ lse, const float *__restrict__ Dr,
                                                          float *dq, int acc_q, float *__restrict__ dqpart, const float *__restrict__ rot) {
  using IO = TileIO<KT>;
  __shared__ __attribute__((aligned(16))) float sK[KT * LD];
  __shared__ __attribute__((aligned(16))) float sV[KT * LD];
  __shared__ __attribute__((aligned(16))) float sKt[HD * IO::LDT];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, g = lane / 32, l32 = lane % 32;
  const int nhb = p.Hq * p.B;
  const int sp = (int)(blockIdx.x % p.splits);
  const unsigned bid = blockIdx.x / p.splits;
  const int qtile = (int)((p.T + 127) / 128) - 1 - (int)(bid / nhb);
  const int h = (bid % nhb) % p.Hq, b = (bid % nhb) / p.Hq;
  const int kvh = h / (p.Hq / p.Hkv);
  const size_t qstr = (size_t)p.Hq * HD, kstr = (size_t)p.Hkv * HD;
  const int tq0 = qtile * 128 + wave * 32, t = tq0 + l32;
  const int tq1 = min(tq0 + 31, p.T - 1);
  const bool tv = t < p.T;
  const float *kb = k + (size_t)b * p.T * kstr + (size_t)kvh * HD;
  const float *vb = v + (size_t)b * p.T * kstr + (size_t)kvh * HD;
  const size_t qoff = ((size_t)b * p.T + (tv ? t : 0)) * qstr + (size_t)h * HD;
  float qreg[HD / 2], greg[HD / 2];
  load_row_regs(qreg, q + qoff, tv, g, p.c2);
  load_row_regs(greg, go + qoff, tv, g, 1.0f);
  const size_t sidx = ((size_t)b * p.Hq + h) * p.T + (tv ? t : 0);
  const float L2 = tv ? lse[sidx] : 0.f, Dt = tv ? Dr[sidx] : 0.f;
  const int lo_t = win_lo_m(t, p.window);
  int kt_lo = win_lo_m(qtile * 128, p.window) / KT;
  int kt_hi = min(p.T - 1, qtile * 128 + 127) / KT;
  if (p.splits > 1) {                      // this workgroup's share of the key stages (possibly none)
    const int n = kt_hi - kt_lo + 1, first = kt_lo;
    kt_lo = first + sp * n / p.splits;
    kt_hi = first + (sp + 1) * n / p.splits - 1;
  }
  const int wave_lo = win_lo_m(tq0, p.window), wave_lo_last = win_lo_m(tq1, p.window);
  const bool ragged = tq0 + 31 >= p.T;

  v16f dacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) dacc[dt][r] = 0.f;

  v4f pk[IO::PER], pv[IO::PER];
  unsigned koffs[IO::PER];
  IO::offsets(koffs, kstr, tid);
  IO::load(pk, kb + (size_t)kt_lo * KT * kstr, koffs, (unsigned)kstr, p.T - kt_lo * KT, tid);
  IO::load(pv, vb + (size_t)kt_lo * KT * kstr, koffs, (unsigned)kstr, p.T - kt_lo * KT, tid);
  for (int kt = kt_lo; kt <= kt_hi; kt++) {
    __syncthreads();
    IO::store_rows(pk, sK, tid);
    IO::store_t(pk, sKt, tid);
    IO::store_rows(pv, sV, tid);
    __syncthreads();
    if (kt < kt_hi) {
      IO::load(pk, kb + (size_t)(kt + 1) * KT * kstr, koffs, (unsigned)kstr, p.T - (kt + 1) * KT, tid);
      IO::load(pv, vb + (size_t)(kt + 1) * KT * kstr, koffs, (unsigned)kstr, p.T - (kt + 1) * KT, tid);
    }
    if (tq0 >= p.T) continue;
#pragma unroll
    for (int sub = 0; sub < NSUB; sub++) {
      const int k0 = kt * KT + sub * 32;
      if (k0 > tq1 || k0 + 31 < wave_lo) continue;
      v16f s = rows_dot_regs(sK + sub * 32 * LD, qreg, l32, g);
      v16f dp = rows_dot_regs(sV + sub * 32 * LD, greg, l32, g);
      const bool need_mask = ragged || k0 + 31 > tq0 || k0 < wave_lo_last;
      float ds[16];
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float pr = fast_exp2(s[r] - L2);
        if (need_mask) {
          int key = k0 + acc_row(r, g);
          if (!(tv && key <= t && key >= lo_t)) pr = 0.f;
        }
        ds[r] = pr * (dp[r] - Dt) * p.scale;
      }
      t_dot_acc<IO::LDT>(dacc, sKt, sub * 32, ds, l32, g);
    }
  }
  if (!tv) return;
  // (the rotation is linear: rotating every split's partial and summing them is the rotated sum)
  if (p.splits > 1) store_grad_row(dqpart + sp * ((size_t)p.B * p.T * qstr) + qoff, dacc, g, 1.0f, 0, rot, t);
  else store_grad_row(dq + qoff, dacc, g, 1.0f, acc_q, rot, t);
}

// ---- dK, dV ---------------------------------------------------------------------------------------------
#define QT 32      // queries per LDS stage in dK/dV
// KS: the forward kept its scores (sco: one [key][query] 32 x 32 block per (key sub-tile, query stage) of every
// (sequence, head), T a multiple of 128). S is then read back, four 16-byte loads per lane and stage issued a stage
// ahead, instead of recomputed: no key row in registers, no row-major query tile in LDS, three contractions per stage.
// DS: the score gradients are kept (dsb) for the banded dQ product.
// The query / dO tiles are double-buffered in LDS: the tile of stage it+1 is written (from the registers its global loads
// filled during stage it-1) while stage it computes on the other buffer, the loads of stage it+2 follow, and one barrier
// ends the stage. None of that depends on the stage's MFMAs, and it is straight-line code, so it runs under them.
#define DKV_BUF (2 * QT * LD + 2 * HD * (QT + 4) + 2 * QT)        // floats per buffer: sQ, sG, sQt, sGt, lse, D
// PX (head dim 64, kept scores): the three contractions on the bf16 matrix instruction. The Q and dO tiles are the same for the four
// wavefronts of a workgroup, so they are cut into pieces ONCE, by the threads that store them (each thread holds columns d and d + 32
// of one row, whose pieces pair up into words), into three kinds of planes: dO row-major for dP = dO.V^T (this lane's value row is cut
// once per kernel in the same k-slot order), dO and Q transposed, two rows to a word, for dV += P^T.dO and dK += dS^T.Q: the
// contractions read their tile operand as ready MFMA registers, one b128 per piece, and only the probabilities and score gradients are
// cut as they are made. 7 vector instructions per MFMA where every wavefront cutting every tile it read took 12.7; on one box 522-529 us
// per launch against 580-594. The register file is what is left as the limit at two wavefronts per SIMD (255 of 256, nothing in scratch):
// the kept scores of a stage are asked for at its top, not a stage ahead (16 registers: with them 13 spill and the launch takes 589),
// and scheduling barriers keep the operand fetches from being issued all at once. 2 x 37 KB of LDS.
template <bool KS, bool DS, bool PX = false>
__global__ __launch_bounds__(256, WAVES_PER_SIMD) void FN(attn_bwd_dkv_mfma_k)(AttnP p, const float *__restrict__ q, const float *__restrict__ k,
                                                           const float *__restrict__ v, const float *__restrict__ go,
                                                           const float *__restrict__ lse, const float *__restrict__ Dr,
                                                           float *dk, int acc_k, float *dv, int acc_v, float *part,
                                                           float *dsb, const float *__restrict__ sco, const float *__restrict__ rot) {
  using IO = TileIO<QT>;
  extern __shared__ __attribute__((aligned(16))) float dkv_smem[];      // 2 x 35 KB at hd 64, 2 x 69 KB at hd 128
  constexpr int O_G = QT * LD, O_QT = 2 * QT * LD, O_GT = O_QT + HD * IO::LDT, O_L = O_GT + HD * IO::LDT, O_D = O_L + QT;
  // the wavefront's number as a scalar: what follows from it (its keys' offsets, its blocks of the kept scores and of dS) then stays in scalar
  // registers, five vector registers fewer in a kernel that is short of them (the forward got slower by the same change and keeps tid / 64)
  const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64), g = lane / 32, l32 = lane % 32;
  // 1-D grid, key tile slowest: the first key tiles are seen by the most queries and go first. One workgroup
  // per QUERY head: with a kv group larger than one, each head's dK/dV goes to its own slice of the workspace
  // and attn_group_sum adds the slices in head order (a fixed order, so still deterministic); splitting by
  // head is what gives the dispatcher enough similar-sized pieces to fill 256 CUs.
  const int nhb = p.Hq * p.B;
  const int sp = (int)(blockIdx.x % p.splits);
  const unsigned bid = blockIdx.x / p.splits;
  const int ktile = (int)(bid / nhb);
  const int h = (bid % nhb) % p.Hq, b = (bid % nhb) / p.Hq;
  const int group = p.Hq / p.Hkv;
  const int kvh = h / group, hh = h % group;
  const size_t qstr = (size_t)p.Hq * HD, kstr = (size_t)p.Hkv * HD;
  const int sk0 = ktile * 128 + wave * 32, s = sk0 + l32;
  const bool sv = s < p.T;
  const size_t koff = ((size_t)b * p.T + (sv ? s : 0)) * kstr + (size_t)kvh * HD;
  float kreg[KS || PX ? 1 : HD / 2], vreg[PX ? 1 : HD / 2];
  static_assert(!PX || (KS && HD == 64), "dK/dV on pieces: kept scores and head dim 64 only");
  v4u vp[PX ? 4 : 1][3];
  if constexpr (PX) pl_load_row(vp, v + koff, sv, g, 1.0f);
  else {
    if constexpr (!KS) load_row_regs(kreg, k + koff, sv, g, p.c2);
    load_row_regs(vreg, v + koff, sv, g, 1.0f);
  }
  // queries that can see a key of this workgroup: t in [ktile*128, last key + window - 1]
  const int qt_lo = ktile * (128 / QT);
  // With a dS matrix to fill (dsb: T a multiple of 128), the loop runs on to the end of the last 128-row tile whose
  // band of keys (starting at a multiple of 128) still holds this key tile, so that every 32 x 32 block the banded
  // dQ product will read has been written: zeros where no pair is live.
  const int t_last = p.window > 0 ? min(p.T - 1, dsb ? ((ktile * 128 + 126 + p.window) & ~127) + 127 : ktile * 128 + 127 + p.window - 1)
                                  : p.T - 1;
  const int qt_hi = t_last / QT;
  const int nqt = qt_hi - qt_lo + 1;
  const int wave_t_hi = p.window > 0 ? sk0 + 31 + p.window - 1 : p.T - 1;   // last query that sees a key of this wave
  // queries that see this lane's key s: s ... min(T - 1, s + window - 1); as an unsigned span from s (none for a key past the end)
  const unsigned span = sv ? (unsigned)((p.window > 0 ? min(p.T - 1, s + p.window - 1) : p.T - 1) - s) : 0u;
  const unsigned dead = sv ? 0u : 0x40000000u;      // added to every relative index of a key past the end: beyond any span

  v16f kacc[HD / 32], vacc[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) { kacc[dt][r] = 0.f; vacc[dt][r] = 0.f; }

  // this workgroup's share of the query stages
  const int it_lo = p.splits > 1 ? sp * nqt / p.splits : 0;
  const int niter = p.splits > 1 ? (sp + 1) * nqt / p.splits : nqt;
  // ONE_SET (head dim 128 without kept scores, where both operand rows sit in registers): one set of staging registers
  // serves the Q and the dO tile in turn, which keeps the kernel inside the register file. The Q tile of stage it+1 is
  // in flight from the end of stage it-1 and written in the middle of stage it; the dO tile is loaded there and written
  // at the stage's end, where the Q tile of stage it+2 is asked for.
  constexpr bool ONE_SET = HD >= 128 && !KS;
  v4f pq[IO::PER], pg[ONE_SET ? 1 : IO::PER], psc[KS ? 4 : 1];
  float pstat = 0.f;
  // this wavefront's block of kept scores for a query stage: lane = key row of the block, queries 8a + 4g + (0..3)
  const float *scw = KS ? sco + (((size_t)b * p.Hq + h) * (p.T / 32) + sk0 / 32) * (p.T / 32) * 1024 + l32 * 32 + 4 * g : nullptr;
  const float *qb = q + (size_t)b * p.T * qstr + (size_t)h * HD;
  const float *gb = go + (size_t)b * p.T * qstr + (size_t)h * HD;
  // row statistics of a stage: threads 0..31 fetch lse, 32..63 fetch D (the other threads fetch the same words again: no branch)
  const float *statp = ((tid & QT) ? Dr : lse) + ((size_t)b * p.Hq + h) * p.T;
  unsigned qoffs[IO::PER];
  if constexpr (PX) {          // row tid / 8: columns 4 (tid % 8) + (0..3), and 32 further on in the second unit
    qoffs[0] = (unsigned)(((tid / 8) * qstr + 4 * (tid % 8)) * sizeof(float));
    qoffs[IO::PER - 1] = qoffs[0] + 32 * (unsigned)sizeof(float);
  } else IO::offsets(qoffs, qstr, tid);
  // Stage indices past the end are clamped to the last stage: its tile is loaded, and written to the idle buffer, again,
  // which nobody reads; the loop body has no test for "is there a next stage".
  // With kept scores T is a multiple of 128 and no tile is short: telling the loads so takes their clamp arithmetic out of the
  // stage (measured: 1 % at head dim 128, where the kernel is short of registers; nothing at 64, where it stays as it was).
  constexpr bool WHOLE = KS && HD >= 128;
  auto load_q = [&](int it) {
    const int qt = qt_lo + min(it, niter - 1);
    IO::load(pq, qb + (size_t)qt * QT * qstr, qoffs, (unsigned)qstr, WHOLE || PX ? QT : p.T - qt * QT, tid);
  };
  auto load_g = [&](int it) {          // dO and the row statistics
    const int qt = qt_lo + min(it, niter - 1);
    if constexpr (ONE_SET) IO::load(pq, gb + (size_t)qt * QT * qstr, qoffs, (unsigned)qstr, p.T - qt * QT, tid);
    else IO::load(pg, gb + (size_t)qt * QT * qstr, qoffs, (unsigned)qstr, WHOLE || PX ? QT : p.T - qt * QT, tid);
    pstat = statp[WHOLE || PX ? qt * QT + (tid % QT) : min(qt * QT + (tid % QT), p.T - 1)];
  };
  auto load_scores = [&](int it) {          // blocks the forward has not written hold anything: their stage is skipped
    const int qt = qt_lo + min(it, niter - 1);
#pragma unroll
    for (int a = 0; a < 4; a++) psc[a] = *reinterpret_cast<const v4f *>(scw + (size_t)qt * 1024 + 8 * a);
  };
  auto store_q = [&](float *buf) {
    if constexpr (PX) {
      unsigned w[3][4];
      pl_cut_unit(pq[0], pq[IO::PER - 1], w);
      pl_store_t(w, reinterpret_cast<unsigned *>(buf) + PL_QT, tid);
      return;
    }
    if (!KS) IO::store_rows(pq, buf, tid);
    IO::store_t(pq, buf + O_QT, tid);
  };
  auto store_g = [&](float *buf) {
    if constexpr (PX) {          // one cut serves both layouts
      unsigned w[3][4];
      pl_cut_unit(pg[0], pg[IO::PER - 1], w);
      pl_store_rows(w, reinterpret_cast<unsigned *>(buf) + PL_GR, tid);
      pl_store_t(w, reinterpret_cast<unsigned *>(buf) + PL_GT, tid);
      if (tid < 2 * QT) buf[PL_L + tid] = pstat;
      return;
    }
    if constexpr (ONE_SET) {
      IO::store_rows(pq, buf + O_G, tid);
      IO::store_t(pq, buf + O_GT, tid);
    } else {
      IO::store_rows(pg, buf + O_G, tid);
      IO::store_t(pg, buf + O_GT, tid);
    }
    if (tid < 2 * QT) buf[O_L + tid] = pstat;           // lse, then D
  };
  // the middle of a stage: the next stage's tile(s) into the idle buffer; its end: what is left of them, and the next loads
  auto stage_middle = [&](float *nxt, int it) {
    store_q(nxt);
    if constexpr (ONE_SET) load_g(it + 1);
    else store_g(nxt);
  };
  auto stage_end = [&](float *nxt, int it) {
    if constexpr (ONE_SET) {
      store_g(nxt);
      load_q(it + 2);
    }
  };
  if (it_lo < niter) {
    load_q(it_lo);
    if constexpr (ONE_SET) {
      store_q(dkv_smem);
      load_g(it_lo);
      store_g(dkv_smem);
      load_q(it_lo + 1);
    } else {
      load_g(it_lo);
      if (KS && !PX) load_scores(it_lo);
      store_q(dkv_smem);
      store_g(dkv_smem);
      load_q(it_lo + 1);
      load_g(it_lo + 1);
    }
    __syncthreads();
  }
  for (int it = it_lo; it < niter; it++) {
    constexpr int BUF = PX ? PL_BUF : DKV_BUF;
    const float *cur = dkv_smem + ((it - it_lo) & 1) * BUF;
    float *nxt = dkv_smem + (((it - it_lo) & 1) ^ 1) * BUF;
    const float *sQ = cur, *sG = cur + O_G, *sQt = cur + O_QT, *sGt = cur + O_GT, *sL = cur + (PX ? PL_L : O_L), *sD = cur + (PX ? PL_L + QT : O_D);
    const unsigned *pl = reinterpret_cast<const unsigned *>(cur);
    v16f sc;
    if (KS) {            // out of the prefetch registers, which the next stage's scores then fill
      if constexpr (PX) load_scores(it);          // (on pieces there are no registers for a stage of look-ahead: asked for here, first used after the dP contraction)
#pragma unroll
      for (int r = 0; r < 16; r++) sc[r] = psc[r / 4][r % 4];
      if constexpr (!PX) load_scores(it + 1);
    }
    const int t0 = (qt_lo + it) * QT;
    // this lane's column of the dS block of (query stage, keys of this wavefront): rows t0 + 8a + 4g + j. The matrix of a
    // (sequence, head) is kept as [row tile of 128][key step of 32][128 rows][32 keys]: a wavefront's block is 4 KB in one piece
    float *dsc = DS ? dsb + ((((size_t)b * p.Hq + h) * (unsigned)(p.T / 128) + (unsigned)t0 / 128) * (unsigned)(p.T / 32) + (unsigned)sk0 / 32) * 4096 +
                          ((unsigned)t0 % 128 + 4 * g) * 32 + l32
                    : nullptr;
    if (t0 + 31 < sk0 || t0 > wave_t_hi || sk0 >= p.T) {             // wave-uniform: no (query, key) pair of this tile is live
      if (DS) {
#pragma unroll
        for (int r = 0; r < 16; r++) dsc[(8 * (r / 4) + r % 4) * 32] = 0.f;
      }
      stage_middle(nxt, it);
      if constexpr (!ONE_SET) {
        load_q(it + 2);
        load_g(it + 2);
      }
    } else {
      // at head dim 128 without kept scores both operand rows live in registers (128 of them): four LDS reads in flight
      // instead of eight keep the kernel inside the register file
      constexpr int DKV_NB = (HD >= 128 && !KS) ? 4 : 8;
      if constexpr (!KS) {
        sc = rows_dot_regs<DKV_NB>(sQ, kreg, l32, g);
      }
      // The stage as straight-line code. A pair (query tq, key s) is live when s <= tq <= last query that sees s: one
      // unsigned compare per element against this lane's span (computed once per kernel), applied to every tile: a
      // wave-uniform "does this tile need a mask" test would cut the stage into basic blocks, and the scheduler cannot
      // move an instruction across those. Order: the probabilities need the scores only, so their exponentials are written
      // between the issue of the dP contraction and its first use, and the dV contraction (which needs the probabilities
      // only) between dP and the dS arithmetic: the vector ALU work has independent MFMAs to run under instead of sitting
      // between two dependent blocks, and the group barriers ask for that interleaving (one MFMA, a few vector
      // instructions, and again).
      v16f dp;
      if constexpr (PX) dp = pl_rows_dot(pl + PL_GR, vp, l32, g);
      else dp = rows_dot_regs<DKV_NB>(sG, vreg, l32, g);
      float pr[16], ds[16];
      const unsigned rel0 = (unsigned)(t0 + 4 * g - s) + dead;          // query index relative to this lane's key, element (a, j) adds 8a + j
#pragma unroll
      for (int a = 0; a < 4; a++) {
        v4f lv = *reinterpret_cast<const v4f *>(sL + 8 * a + 4 * g);
#pragma unroll
        for (int j = 0; j < 4; j++) {
          float e = fast_exp2(sc[4 * a + j] - lv[j]);
          pr[4 * a + j] = (rel0 + (unsigned)(8 * a + j)) <= span ? e : 0.f;
        }
      }
      if constexpr (!PX) {
#pragma unroll
        for (int i = 0; i < HD / 2; i++) {          // dP with the exponentials
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        }
      }
      if constexpr (PX) pl_t_dot(vacc, pl + PL_GT, pr, l32, g);
      else t_dot_acc<IO::LDT, DKV_NB>(vacc, sGt, 0, pr, l32, g);
#pragma unroll
      for (int a = 0; a < 4; a++) {
        v4f dv4 = *reinterpret_cast<const v4f *>(sD + 8 * a + 4 * g);
#pragma unroll
        for (int j = 0; j < 4; j++) ds[4 * a + j] = pr[4 * a + j] * (dp[4 * a + j] - dv4[j]) * p.scale;
      }
      if constexpr (!PX) {
#pragma unroll
        for (int i = 0; i < HD / 2; i++) {          // dV with the dS arithmetic
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
        }
      }
      // next stage's tile into the idle buffer (its loads were issued a stage ago), this stage's dS out, the loads of the
      // stage after next: all independent of the dK contraction that follows
      stage_middle(nxt, it);
      if (DS) {
#pragma unroll
        for (int r = 0; r < 16; r++) dsc[(8 * (r / 4) + r % 4) * 32] = ds[r];
      }
      if constexpr (!ONE_SET) {
        load_q(it + 2);
        load_g(it + 2);
      }
      if constexpr (PX) pl_t_dot(kacc, pl + PL_QT, ds, l32, g);
      else t_dot_acc<IO::LDT, DKV_NB>(kacc, sQt, 0, ds, l32, g);
    }
    stage_end(nxt, it);
    __syncthreads();
  }
  if (sv) {
    if (part) {            // slice (split, head of the group) of the workspace, same [row][Hkv*hd] layout as dk
      const size_t slice = (size_t)p.B * p.T * kstr;
      const int nslice = p.splits * group, mine = sp * group + hh;
      store_grad_row(part + (size_t)mine * slice + koff, kacc, g, 1.0f, 0, rot, s);      // every slice rotated: their sum is the rotated sum
      store_row(part + (size_t)(nslice + mine) * slice + koff, vacc, g, 1.0f, 0);
    } else {
      store_grad_row(dk + koff, kacc, g, 1.0f, acc_k, rot, s);
      store_row(dv + koff, vacc, g, 1.0f, acc_v);
    }
  }
}

// dk (+)= sum of its slices (splits x heads of the group), in slice order; same for dv
__global__ __launch_bounds__(256) void FN(attn_group_sum)(const float *__restrict__ part, int group, size_t n4, float *dk, int acc_k,
                                                      float *dv, int acc_v) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  const v4f *pp = reinterpret_cast<const v4f *>(part);
  v4f sk = pp[i], sv = pp[(size_t)group * n4 + i];
  for (int hh = 1; hh < group; hh++) { sk += pp[(size_t)hh * n4 + i]; sv += pp[(size_t)(group + hh) * n4 + i]; }
  v4f *ok = reinterpret_cast<v4f *>(dk) + i, *ov = reinterpret_cast<v4f *>(dv) + i;
  *ok = acc_k ? *ok + sk : sk;
  *ov = acc_v ? *ov + sv : sv;
}

#define DKV_SMEM (2 * DKV_BUF * sizeof(float))

// fpart: workspace for the split partials (splits x output, then splits x rows maxima, splits x rows sums), or null
// sco: where to keep the scores for the backward (B*Hq*T*T floats, T a multiple of 128), or null
int FN(attn_fwd_mfma)(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf out, gt_buf lse, float *fpart, float *sco) {
  GT_REQUIRE(ctx, (q | k | v | out) % 16 == 0, "attention: buffers must be 16-byte aligned");
  GT_REQUIRE(ctx, p.splits >= 1 && (p.splits == 1 || fpart), "attention: split forward without a workspace");
  if (!(ctx->attn_smem_set & (HD << 8))) {   // once per context (device): more than the 64 KB a kernel gets by default
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_fwd_mfma_k)<false>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)FWD_SMEM));
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_fwd_mfma_k)<true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)FWD_SMEM));
    ctx->attn_smem_set |= HD << 8;
  }
  dim3 grid((unsigned)(cdiv(p.T, 128) * p.Hq * p.B * p.splits));
#if HD == 64 || HD == 128
  if (ctx->opt_attn_pieces) {          // "attn.split_bf16": the forward of head dims 64 and 128 on the bf16 matrix instruction
    if (!(ctx->attn_smem_set & (1 << 20))) {
      GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_fwd_mfma_k)<false, true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)FWD_SMEM));
      GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_fwd_mfma_k)<true, true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)FWD_SMEM));
      ctx->attn_smem_set |= 1 << 20;
    }
    if (sco)
      hipLaunchKernelGGL((FN(attn_fwd_mfma_k)<true, true>), grid, dim3(256), FWD_SMEM, ctx->stream, p, P<const float>(q), P<const float>(k),
                         P<const float>(v), P<float>(out), P<float>(lse), fpart, sco);
    else
      hipLaunchKernelGGL((FN(attn_fwd_mfma_k)<false, true>), grid, dim3(256), FWD_SMEM, ctx->stream, p, P<const float>(q), P<const float>(k),
                         P<const float>(v), P<float>(out), P<float>(lse), fpart, sco);
    GT_LAUNCHED(ctx);
    return 0;
  }
#endif
  if (sco)
    hipLaunchKernelGGL(FN(attn_fwd_mfma_k)<true>, grid, dim3(256), FWD_SMEM, ctx->stream, p, P<const float>(q), P<const float>(k),
                       P<const float>(v), P<float>(out), P<float>(lse), fpart, sco);
  else
    hipLaunchKernelGGL(FN(attn_fwd_mfma_k)<false>, grid, dim3(256), FWD_SMEM, ctx->stream, p, P<const float>(q), P<const float>(k),
                       P<const float>(v), P<float>(out), P<float>(lse), fpart, sco);
  GT_LAUNCHED(ctx);
  return 0;
}

// Dr: the per-row sums D; part: workspace for the dK/dV slices (2 * splits * group slices of B*T*Hkv*hd floats) or
// null when there is one slice; dqpart: workspace for the dQ partials (splits x dq) or null when splits == 1
// dsb: workspace for the B*Hq [T][T] dS matrices, or null. With it dK/dV writes dS as it goes and dQ is one banded
// product dS.K afterwards (5 contractions in all); without it dQ recomputes S and dP in its own kernel (7).
int FN(attn_bwd_mfma)(gt_ctx *ctx, const AttnP &p, gt_buf q, gt_buf k, gt_buf v, gt_buf dout, gt_buf lse, const float *Dr,
                      float *part, float *dqpart, float *dsb, const float *sco, gt_buf dq, int acc_q, gt_buf dk, int acc_k, gt_buf dv,
                      int acc_v, const float *rot_q, const float *rot_k, float *bandp, int band_splits) {
  GT_REQUIRE(ctx, (q | k | v | dout | dq | dk | dv) % 16 == 0, "attention: buffers must be 16-byte aligned");
  const int group = p.Hq / p.Hkv;
  GT_REQUIRE(ctx, p.splits >= 1 && (p.splits == 1 || dqpart || dsb) && (p.splits * group == 1 || part),
             "attention: split backward without a workspace");
  GT_REQUIRE(ctx, !sco || (p.T % 128 == 0 && HD >= 64), "attention: kept scores with an unsupported shape");
  if (!(ctx->attn_smem_set & HD)) {   // once per context (device): more than the 64 KB a kernel gets by default at hd 128
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_bwd_dkv_mfma_k)<false, false>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)DKV_SMEM));
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_bwd_dkv_mfma_k)<false, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)DKV_SMEM));
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_bwd_dkv_mfma_k)<true, false>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)DKV_SMEM));
    GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_bwd_dkv_mfma_k)<true, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)DKV_SMEM));
    ctx->attn_smem_set |= HD;
  }
  GT_REQUIRE(ctx, !dsb || (p.T % 128 == 0 && HD >= 64), "attention: dS workspace with an unsupported shape");
  if (!dsb) {
    ProfScope ps(ctx, "attention.bwd.dq");
    dim3 grid((unsigned)(cdiv(p.T, 128) * p.Hq * p.B * p.splits));
    hipLaunchKernelGGL(FN(attn_bwd_dq_mfma_k), grid, dim3(256), 0, ctx->stream, p, P<const float>(q), P<const float>(k),
                       P<const float>(v), P<const float>(dout), P<const float>(lse), Dr, P<float>(dq), acc_q, dqpart, rot_q);
    GT_LAUNCHED(ctx);
  }
  {
    ProfScope ps(ctx, "attention.bwd.dkv");
    dim3 grid((unsigned)(cdiv(p.T, 128) * p.Hq * p.B * p.splits));
    size_t smem = DKV_SMEM;
    auto launch = [&](auto kern) {
      hipLaunchKernelGGL(kern, grid, dim3(256), smem, ctx->stream, p, P<const float>(q), P<const float>(k), P<const float>(v),
                         P<const float>(dout), P<const float>(lse), Dr, P<float>(dk), acc_k, P<float>(dv), acc_v, part, dsb, sco, rot_k);
    };
#if HD == 64
    if (ctx->opt_attn_pieces && sco) {          // "attn.split_bf16": dK/dV of head dim 64 on the bf16 matrix instruction, where the forward kept
                                                // its scores (recomputing them needs the key row's pieces too: 34-37 registers spilled)
      if (!(ctx->attn_smem_set & (1 << 21))) {
        GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_bwd_dkv_mfma_k)<true, false, true>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * PL_BUF * sizeof(unsigned))));
        GT_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(FN(attn_bwd_dkv_mfma_k)<true, true, true>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * PL_BUF * sizeof(unsigned))));
        ctx->attn_smem_set |= 1 << 21;
      }
      smem = 2 * PL_BUF * sizeof(unsigned);
      dsb ? launch(FN(attn_bwd_dkv_mfma_k)<true, true, true>) : launch(FN(attn_bwd_dkv_mfma_k)<true, false, true>);
    } else
#endif
    if (sco) dsb ? launch(FN(attn_bwd_dkv_mfma_k)<true, true>) : launch(FN(attn_bwd_dkv_mfma_k)<true, false>);
    else dsb ? launch(FN(attn_bwd_dkv_mfma_k)<false, true>) : launch(FN(attn_bwd_dkv_mfma_k)<false, false>);
    GT_LAUNCHED(ctx);
    if (part) {
      size_t n4 = (size_t)p.B * p.T * p.Hkv * HD / 4;
      hipLaunchKernelGGL(FN(attn_group_sum), dim3((unsigned)cdiv((int64_t)n4, 256)), dim3(256), 0, ctx->stream, part, p.splits * group, n4,
                         P<float>(dk), acc_k, P<float>(dv), acc_v);
      GT_LAUNCHED(ctx);
    }
  }
  if (dsb) {
    ProfScope ps(ctx, "attention.bwd.dq");
    if (gemm_band_dq(ctx, p.B, p.T, p.Hq, p.Hkv, HD, p.window, dsb, P<const float>(k), P<float>(dq), acc_q, rot_q, bandp, band_splits)) return 1;
  }
  return 0;
}
