// matmul_f32_mfma.hip -- hand-written CDNA4 (gfx950) matmul template for fp32 operands.
//
// C[z][m][n] = epilogue( sum_k A(z,m,k) * B(z,k,n) ) with fp32 inputs, exact fp32
// products and fp32 accumulation on v_mfma_f32_32x32x2_f32 (157 TFLOP/s dense peak).
// Same configuration block as the 16-bit template (templates.cc prepends it):
//
//   POLY_M/N/K/Z        problem sizes; K % 16 == 0
//   POLY_BM/BN          workgroup tile (multiples of 32 * waves); POLY_WAVES_M x POLY_WAVES_N waves
//   POLY_A_KC/B_KC      1: operand contiguous along K (16-byte loads along K);
//                       0: contiguous along its row axis (16-byte loads along that axis,
//                       written to LDS as four single floats)
//   POLY_A_PTR/B_PTR, poly_a_row(m), poly_b_row(n), poly_a_z(z), poly_b_z(z), poly_a_k(k), poly_b_k(k)
//   POLY_SIGNATURE, POLY_EPILOGUE(acc, m, n, z)
//   POLY_GEN            1: the operands are expressions, not arrays.  Then instead of the
//                       pointer/offset items above:
//                         POLY_A_NLOADS, POLY_A_LOAD(m, k, z, raw)  fetches what element
//                           A(z,m,k) is computed from into `unsigned int raw[POLY_A_NLOADS]`
//                         POLY_A_MATH(m, k, z, raw)  the element as a float
//                       (same for B with n), K may be any size (elements past K are 0), and
//                       POLY_A_KC/B_KC only choose which way consecutive threads walk.
//                       Fetches run ahead in the register ring like the plain loads; the
//                       arithmetic happens on the way to LDS.
//   POLY_PF_DEPTH       K tiles the global loads run ahead (default 4)
//   POLY_KSPLIT         S > 1: the K tiles are dealt to S workgroups per output tile
//                       (blockIdx.y = z * S + s; S divides the number of K tiles) and the
//                       accumulators go to poly_scratch[s][z][m][n] (fp32) for a second
//                       kernel to add up and finish; for deep products with few tiles
//
// Data path: global --16B loads, four K tiles ahead--> registers --> LDS [row][16 k]
// (rows padded to 20 floats: 16-byte fragment reads of 16 consecutive rows then fall on
// different banks), double buffered.  The 32x32x2 MFMA takes one k per half-wave: lane l supplies
// A[l % 32][k(l / 32)] and B[k(l / 32)][l % 32].  The k index is only summed over, so
// the four MFMAs of an 8-deep chunk let half-wave h supply k = 4 h + s (s = 0..3): a lane
// then needs four consecutive k of its row, ONE 16-byte LDS read per operand and chunk.
#ifdef POLY_TEMPLATE_STANDALONE
#include <hip/hip_runtime.h>
#define POLY_M 4096
#define POLY_N 512
#define POLY_K 784
#define POLY_Z 1
#define POLY_BM 128
#define POLY_BN 128
#define POLY_WAVES_M 2
#define POLY_WAVES_N 2
#define POLY_GROUP_M 8
#define POLY_A_KC 1
#define POLY_B_KC 1
#define POLY_A_PTR data1
#define POLY_B_PTR data2
__device__ __forceinline__ int poly_a_row(int m) { return m * POLY_K; }
__device__ __forceinline__ int poly_b_row(int n) { return n * POLY_K; }
__device__ __forceinline__ int poly_a_z(int z) { return 0; }
__device__ __forceinline__ int poly_b_z(int z) { return 0; }
__device__ __forceinline__ int poly_a_k(int k) { return k; }
__device__ __forceinline__ int poly_b_k(int k) { return k; }
#define POLY_SIGNATURE float *data0, const float *__restrict__ data1, const float *__restrict__ data2
#define POLY_EPILOGUE(acc, m, n, z) data0[(m) * POLY_N + (n)] = (acc)
#endif

typedef float pf_f32x4 __attribute__((ext_vector_type(4)));
typedef pf_f32x4 pf_f32x4_u __attribute__((aligned(4)));
typedef float pf_acc16 __attribute__((ext_vector_type(16)));

#define PF_BK 16
#define PF_LDK 20
#define PF_WM (POLY_BM / POLY_WAVES_M)
#define PF_WN (POLY_BN / POLY_WAVES_N)
#define PF_TM (PF_WM / 32)
#define PF_TN (PF_WN / 32)
#define PF_NTHREADS (64 * POLY_WAVES_M * POLY_WAVES_N)
#ifndef POLY_GEN
#define POLY_GEN 0
#endif
#ifndef POLY_PF_DEPTH
#define POLY_PF_DEPTH 4
#endif
#ifndef POLY_KSPLIT
#define POLY_KSPLIT 1
#endif
#define PF_KT (((POLY_K + PF_BK - 1) / PF_BK) / POLY_KSPLIT)

// Staging of one operand tile (ROWS x 16 floats): 16-byte pieces, ROWS * 4 of them.
template <int ROWS, bool KC>
struct PfStage {
  static constexpr int PIECES = ROWS * 4;
  static constexpr int NL = (PIECES + PF_NTHREADS - 1) / PF_NTHREADS;
  // K-contiguous: piece c = (row c / 4, k chunk c % 4); row-contiguous: (k c / (ROWS/4), row chunk c % (ROWS/4))
  static __device__ __forceinline__ bool active(int i) { return PIECES % PF_NTHREADS == 0 || (int)threadIdx.x + i * PF_NTHREADS < PIECES; }
  static __device__ __forceinline__ int row_of(int i) {
    const int c = threadIdx.x + i * PF_NTHREADS;
    return KC ? c / 4 : (c % (ROWS / 4)) * 4;
  }
  static __device__ __forceinline__ int k_of(int i) {
    const int c = threadIdx.x + i * PF_NTHREADS;
    return KC ? (c % 4) * 4 : c / (ROWS / 4);
  }
  static __device__ __forceinline__ void store(float *lds, const pf_f32x4 (&regs)[NL]) {
#pragma unroll
    for (int i = 0; i < NL; i++) {
      if (!active(i)) continue;
      const int row = row_of(i), k = k_of(i);
      if (KC) {
        *(pf_f32x4 *)(lds + row * PF_LDK + k) = regs[i];
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) lds[(row + e) * PF_LDK + k] = regs[i][e];
      }
    }
  }
};

#if POLY_GEN
#define PF_A_NRAW POLY_A_NLOADS
#define PF_B_NRAW POLY_B_NLOADS
#endif

extern "C" __global__ void __launch_bounds__(PF_NTHREADS) poly_k(POLY_SIGNATURE) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][POLY_BM * PF_LDK];
  __shared__ __attribute__((aligned(16))) float lds_b[2][POLY_BN * PF_LDK];

  // Tile coordinates: ids congruent mod 8 (one XCD, one L2) form a contiguous run of
  // tiles; within a run, bands of POLY_GROUP_M tile rows are walked along N.
  constexpr int TILES_M = (POLY_M + POLY_BM - 1) / POLY_BM;
  constexpr int TILES_N = (POLY_N + POLY_BN - 1) / POLY_BN;
  constexpr int NT = TILES_M * TILES_N;
  int bid = blockIdx.x;
  {
    constexpr int PER = NT / 8, REM = NT % 8;
    const int xcd = bid & 7, idx = bid >> 3;
    bid = (xcd < REM ? xcd * (PER + 1) : REM * (PER + 1) + (xcd - REM) * PER) + idx;
  }
  int tile_m, tile_n;
  {
    constexpr int GM = POLY_GROUP_M;
    const int per_group = GM * TILES_N;
    const int group = bid / per_group, first_m = group * GM;
    const int gsz = (TILES_M - first_m) < GM ? (TILES_M - first_m) : GM;
    const int in_group = bid - group * per_group;
    tile_m = first_m + in_group % gsz;
    tile_n = in_group / gsz;
  }
  const int z = blockIdx.y / POLY_KSPLIT;
  const int kt_base = (blockIdx.y % POLY_KSPLIT) * PF_KT;      // first K tile of this workgroup's share
  const int m0 = tile_m * POLY_BM, n0 = tile_n * POLY_BN;
  typedef PfStage<POLY_BM, POLY_A_KC != 0> StageA;
  typedef PfStage<POLY_BN, POLY_B_KC != 0> StageB;
  // Global loads run PF_DEPTH K tiles ahead of the math, in a ring of register sets (tile t
  // in set t % PF_DEPTH): with one small workgroup per CU nothing else hides their latency.
  constexpr int PF_DEPTH = POLY_PF_DEPTH;
#if POLY_GEN
  // element e of piece i: (row + e, k) for row-walking pieces, (row, k + e) for k-walking
  // ones; rows past the edge are clamped (computed, never stored), k past the end gives 0
  unsigned int ra[PF_DEPTH][StageA::NL][4][PF_A_NRAW], rb[PF_DEPTH][StageB::NL][4][PF_B_NRAW];
  auto a_coord = [&](int kt, int i, int e, int *m, int *k) {
    const int row = m0 + StageA::row_of(i) + (POLY_A_KC ? 0 : e);
    *m = row < POLY_M ? row : POLY_M - 1;
    *k = (kt_base + kt) * PF_BK + StageA::k_of(i) + (POLY_A_KC ? e : 0);
  };
  auto b_coord = [&](int kt, int i, int e, int *n, int *k) {
    const int row = n0 + StageB::row_of(i) + (POLY_B_KC ? 0 : e);
    *n = row < POLY_N ? row : POLY_N - 1;
    *k = (kt_base + kt) * PF_BK + StageB::k_of(i) + (POLY_B_KC ? e : 0);
  };
  auto load_tiles = [&](int kt, int set) {
#pragma unroll
    for (int i = 0; i < StageA::NL; i++)
      if (StageA::active(i)) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          int m, k;
          a_coord(kt, i, e, &m, &k);
#pragma unroll
          for (int j = 0; j < PF_A_NRAW; j++) ra[set][i][e][j] = 0u;
          if (POLY_K % PF_BK == 0 || k < POLY_K) { POLY_A_LOAD(m, k, z, ra[set][i][e]); }
        }
      }
#pragma unroll
    for (int i = 0; i < StageB::NL; i++)
      if (StageB::active(i)) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          int n, k;
          b_coord(kt, i, e, &n, &k);
#pragma unroll
          for (int j = 0; j < PF_B_NRAW; j++) rb[set][i][e][j] = 0u;
          if (POLY_K % PF_BK == 0 || k < POLY_K) { POLY_B_LOAD(n, k, z, rb[set][i][e]); }
        }
      }
  };
  auto store_tiles = [&](int kt, int set, int buf) {
    pf_f32x4 va[StageA::NL], vb[StageB::NL];
#pragma unroll
    for (int i = 0; i < StageA::NL; i++)
      if (StageA::active(i)) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          int m, k;
          a_coord(kt, i, e, &m, &k);
          va[i][e] = (POLY_K % PF_BK == 0 || k < POLY_K) ? POLY_A_MATH(m, k, z, ra[set][i][e]) : 0.0f;
        }
      }
#pragma unroll
    for (int i = 0; i < StageB::NL; i++)
      if (StageB::active(i)) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          int n, k;
          b_coord(kt, i, e, &n, &k);
          vb[i][e] = (POLY_K % PF_BK == 0 || k < POLY_K) ? POLY_B_MATH(n, k, z, rb[set][i][e]) : 0.0f;
        }
      }
    StageA::store(lds_a[buf], va);
    StageB::store(lds_b[buf], vb);
  };
#else
  const float *__restrict__ gA = POLY_A_PTR + poly_a_z(z);
  const float *__restrict__ gB = POLY_B_PTR + poly_b_z(z);
  pf_f32x4 ra[PF_DEPTH][StageA::NL], rb[PF_DEPTH][StageB::NL];
  // Per-thread global offsets of the rows this thread stages.  Rows past the edge are
  // clamped to the last valid row (or row group): loaded and multiplied, never stored.
  int a_off[StageA::NL], b_off[StageB::NL];
#pragma unroll
  for (int i = 0; i < StageA::NL; i++) {
    const int row = m0 + StageA::row_of(i);
    a_off[i] = poly_a_row(POLY_A_KC ? (row < POLY_M ? row : POLY_M - 1) : (row + 3 < POLY_M ? row : POLY_M - 4));
  }
#pragma unroll
  for (int i = 0; i < StageB::NL; i++) {
    const int row = n0 + StageB::row_of(i);
    b_off[i] = poly_b_row(POLY_B_KC ? (row < POLY_N ? row : POLY_N - 1) : (row + 3 < POLY_N ? row : POLY_N - 4));
  }
  auto load_tiles = [&](int kt, int set) {
    const int k0 = (kt_base + kt) * PF_BK;
#pragma unroll
    for (int i = 0; i < StageA::NL; i++)
      if (StageA::active(i)) ra[set][i] = *(const pf_f32x4_u *)(gA + a_off[i] + poly_a_k(k0 + StageA::k_of(i)));
#pragma unroll
    for (int i = 0; i < StageB::NL; i++)
      if (StageB::active(i)) rb[set][i] = *(const pf_f32x4_u *)(gB + b_off[i] + poly_b_k(k0 + StageB::k_of(i)));
  };
  auto store_tiles = [&](int kt, int set, int buf) {
    (void)kt;
    StageA::store(lds_a[buf], ra[set]);
    StageB::store(lds_b[buf], rb[set]);
  };
#endif

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, half = lane >> 5;
  const int wm = (wave % POLY_WAVES_M) * PF_WM, wn = (wave / POLY_WAVES_M) * PF_WN;
  pf_acc16 acc[PF_TM][PF_TN];
#pragma unroll
  for (int i = 0; i < PF_TM; i++)
#pragma unroll
    for (int j = 0; j < PF_TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

#pragma unroll
  for (int d = 0; d < PF_DEPTH; d++)
    if (d < PF_KT) load_tiles(d, d);
  store_tiles(0, 0, 0);
  if (PF_DEPTH < PF_KT) load_tiles(PF_DEPTH, 0);
  __syncthreads();
  for (int kt0 = 0; kt0 < PF_KT; kt0 += PF_DEPTH) {
#pragma unroll
    for (int d = 0; d < PF_DEPTH; d++) {
      const int kt = kt0 + d;
      if (kt >= PF_KT) break;
      const int cur = kt & 1;
#pragma unroll
      for (int q = 0; q < PF_BK / 8; q++) {
        // four consecutive k (8 q + 4 half ..) of this lane's rows
        pf_f32x4 fa[PF_TM], fb[PF_TN];
#pragma unroll
        for (int i = 0; i < PF_TM; i++) fa[i] = *(const pf_f32x4 *)(lds_a[cur] + (wm + i * 32 + (lane & 31)) * PF_LDK + 8 * q + 4 * half);
#pragma unroll
        for (int j = 0; j < PF_TN; j++) fb[j] = *(const pf_f32x4 *)(lds_b[cur] + (wn + j * 32 + (lane & 31)) * PF_LDK + 8 * q + 4 * half);
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
          for (int i = 0; i < PF_TM; i++)
#pragma unroll
            for (int j = 0; j < PF_TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
      }
      if (kt + 1 < PF_KT) {
        // tile kt + 1 waits in the next set of the ring; once it is in LDS the set takes tile kt + 1 + PF_DEPTH
        const int nset = (d + 1) % PF_DEPTH;
        store_tiles(kt + 1, nset, cur ^ 1);
        if (kt + 1 + PF_DEPTH < PF_KT) load_tiles(kt + 1 + PF_DEPTH, nset);
      }
      __syncthreads();
    }
  }

  // Accumulator layout of the 32x32 MFMA: register r of lane l holds row
  // 8*(r/4) + 4*(l/32) + r%4, column l%32: the 32 lanes of a half-wave write 32
  // consecutive columns (128 bytes) of a row.
#pragma unroll
  for (int i = 0; i < PF_TM; i++)
#pragma unroll
    for (int j = 0; j < PF_TN; j++) {
      const int n = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
#if POLY_KSPLIT > 1
        if (m < POLY_M && n < POLY_N)
          poly_scratch[(((size_t)(blockIdx.y % POLY_KSPLIT) * POLY_Z + z) * POLY_M + m) * POLY_N + n] = acc[i][j][r];
#else
        if (m < POLY_M && n < POLY_N) { POLY_EPILOGUE(acc[i][j][r], m, n, z); }
#endif
      }
    }
}
