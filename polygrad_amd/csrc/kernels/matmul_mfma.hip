// matmul_mfma.hip -- hand-written CDNA4 (gfx950) matmul template.
//
// C[z][m][n] = epilogue( sum_k A(z,m,k) * B(z,k,n) ) with 16-bit float inputs
// (bf16 or fp16) and fp32 accumulation on the 32x32x16 MFMA.  The renderer
// (templates.cc) instantiates it by prepending a configuration block:
//
//   POLY_TIN            input element type (__bf16 or _Float16)
//   POLY_MFMA(a,b,c)    the MFMA builtin for that type
//   POLY_M/N/K/Z        problem sizes (rows, columns, depth, batch)
//   POLY_BM/BN/BK       workgroup tile; 4 waves as POLY_WM x POLY_WN
//   POLY_A_KC/B_KC      1: operand is contiguous along K in memory (16-byte loads
//                       along K); 0: contiguous along M (resp. N): 16-byte loads
//                       along that axis and a register transpose on the way to LDS
//   POLY_A_PTR/B_PTR    the kernel parameters holding A and B
//   poly_a_row(m), poly_b_row(n), poly_a_z(z), poly_b_z(z), poly_a_k(k), poly_b_k(k)
//                       element offsets contributed by each coordinate
//   POLY_SIGNATURE      the kernel's parameter list
//   POLY_EPILOGUE(acc, m, n, z)   stores one finished element (generated from the
//                       UOps around the REDUCE: casts, bias, activation, index)
//   POLY_KSPLIT         (optional) workgroups sharing the K tiles of one output tile
//   POLY_EP_MID_TYPE, POLY_EP_MID_VALUE(acc, m, n, z), POLY_EP_MID_PTR(m, n, z)
//                       (optional, with POLY_EP_CONTIG) a second output with the layout of the
//                       first: a value the epilogue passes through on its way (the
//                       pre-activation that a backward pass reads), stored as well
//   POLY_EP_CONTIG      1 when consecutive n of a row are consecutive in memory; then
//                       POLY_EP_TYPE, POLY_EP_VALUE(acc, m, n, z) and POLY_EP_PTR(m, n, z)
//                       give the element type, value and address separately and the
//                       template writes 8 values of a row with one store
//   POLY_EP_WIN_BYTES   (optional, set by the epilogue's own code when POLY_EP_WIN_ROOM, the
//                       LDS left beside the operand tiles, suffices) bytes of LDS that
//                       the kernel fills from POLY_EP_WIN_SRC(byte) with the middle of
//                       the epilogue's lookup tables; POLY_EP_VALUE_WIN is then POLY_EP_VALUE
//                       with lookups from there, raising poly_tmax to POLY_WIN_CODES or
//                       more when an input lies outside
//
// Data path: global --16B loads--> registers --(transpose if needed)--> LDS
// [row][K] with padded rows, double buffered; each wave reads 16-byte A and B
// fragments and issues (WM/32)*(WN/32) MFMAs per 16-deep K step.
#ifdef POLY_TEMPLATE_STANDALONE
#include <hip/hip_runtime.h>
#define POLY_TIN __bf16
#define POLY_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)
#define POLY_M 4096
#define POLY_N 4096
#define POLY_K 4096
#define POLY_Z 1
#define POLY_BM 128
#define POLY_BN 128
#define POLY_BK 64
#define POLY_GROUP_M 8
#define POLY_GROUP_ALONG_N 0
#define POLY_PIPE 3
#define POLY_WAVES_M 2
#define POLY_WAVES_N 2
#define POLY_A_KC 1
#define POLY_B_KC 0
#define POLY_A_PTR data1
#define POLY_B_PTR data2
__device__ __forceinline__ int poly_a_row(int m) { return m * POLY_K; }
__device__ __forceinline__ int poly_b_row(int n) { return n; }
__device__ __forceinline__ int poly_a_z(int z) { return 0; }
__device__ __forceinline__ int poly_b_z(int z) { return 0; }
__device__ __forceinline__ int poly_a_k(int k) { return k; }
__device__ __forceinline__ int poly_b_k(int k) { return k * POLY_N; }
#define POLY_SIGNATURE float *data0, const __bf16 *__restrict__ data1, const __bf16 *__restrict__ data2
#define POLY_EPILOGUE(acc, m, n, z) data0[(m) * POLY_N + (n)] = (acc)
#define POLY_EP_CONTIG 1
#define POLY_EP_TYPE float
#define POLY_EP_VALUE(acc, m, n, z) (acc)
#define POLY_EP_PTR(m, n, z) (data0 + (m) * POLY_N + (n))
#endif

typedef POLY_TIN poly_in8 __attribute__((ext_vector_type(8)));
typedef POLY_TIN poly_in4 __attribute__((ext_vector_type(4)));
typedef float poly_acc16 __attribute__((ext_vector_type(16)));
typedef unsigned int poly_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int poly_u32x2 __attribute__((ext_vector_type(2)));
typedef poly_u32x4 poly_u32x4_u __attribute__((aligned(2)));
typedef float poly_f32x4 __attribute__((ext_vector_type(4)));

#define POLY_WM (POLY_BM / POLY_WAVES_M)
#define POLY_WN (POLY_BN / POLY_WAVES_N)
#define POLY_TM (POLY_WM / 32)
#define POLY_TN (POLY_WN / 32)
#define POLY_NTHREADS (64 * POLY_WAVES_M * POLY_WAVES_N)
// LDS tile: [row][BK] with the 16-byte columns of a row XOR-swizzled by the row
// number, so that the 16-byte fragment reads of 8 consecutive rows, the 16-byte
// stores of one row and the 8-byte transposed stores of rows 8 apart all spread
// over the banks without padding.
#define POLY_LDK POLY_BK
#define POLY_NCOL (POLY_BK / 8)
__device__ __forceinline__ int poly_swz(int row) { return (row ^ (row >> 3)) & (POLY_NCOL - 1); }
#ifndef POLY_KSPLIT
#define POLY_KSPLIT 1
#endif
// columns [POLY_N_LO, POLY_N_HI) are this launch's (another launch has the others);
// POLY_N_LO is a multiple of POLY_BN, and so is POLY_N_HI unless it is POLY_N
#ifndef POLY_N_LO
#define POLY_N_LO 0
#define POLY_N_HI POLY_N
#endif
// K tiles one workgroup walks: with POLY_KSPLIT > 1 the K tiles of an output tile are dealt
// to that many workgroups (blockIdx.y = z * POLY_KSPLIT + part), each leaving its fp32
// accumulators where the epilogue macros put them (they may use `poly_ks`, the part).
#ifndef POLY_KT
#define POLY_KT (POLY_K / POLY_BK / POLY_KSPLIT)
#endif
// row pitch (floats) of the 32x32 output staging tile: 16-byte aligned rows, and rows 4
// apart (the two halves of a wave) land on different banks
#define POLY_STAGE_LD 36

// Number of 16-byte global loads per thread for one operand tile.
#define POLY_A_LOADS ((POLY_BM * POLY_BK / 8) / POLY_NTHREADS)
#define POLY_B_LOADS ((POLY_BN * POLY_BK / 8) / POLY_NTHREADS)

// ── K-contiguous operand: thread -> (row, 8-wide k chunk) ──────────────────
// chunks per row = BK/8; consecutive threads walk along K first (full 128-byte
// lines per row when BK = 64).
template <int ROWS, int NLOADS>
struct PolyKC {
  // staging work is cut into UNITS pieces (one 16-byte load and store each) so that the
  // K loop can spread it between its MFMAs
  static constexpr int UNITS = NLOADS;
  static __device__ __forceinline__ void load_unit(const POLY_TIN *__restrict__ base, const int *row_off, int kofs,
                                                   poly_u32x4 (&regs)[NLOADS], int i) {
    const int c = threadIdx.x + i * POLY_NTHREADS;
    const int kc = c % (POLY_BK / 8);
    regs[i] = *(const poly_u32x4_u *)(base + row_off[i] + kofs + kc * 8);
  }
  static __device__ __forceinline__ void store_unit(POLY_TIN *lds, const poly_u32x4 (&regs)[NLOADS], int i) {
    const int c = threadIdx.x + i * POLY_NTHREADS;
    const int row = c / (POLY_BK / 8), kc = c % (POLY_BK / 8);
    *(poly_u32x4 *)(lds + row * POLY_LDK + ((kc ^ poly_swz(row)) * 8)) = regs[i];
  }
  static __device__ __forceinline__ void load(const POLY_TIN *__restrict__ base, const int *row_off, int kofs,
                                              poly_u32x4 (&regs)[NLOADS]) {
#pragma unroll
    for (int i = 0; i < NLOADS; i++) load_unit(base, row_off, kofs, regs, i);
  }
  static __device__ __forceinline__ void store(POLY_TIN *lds, const poly_u32x4 (&regs)[NLOADS]) {
#pragma unroll
    for (int i = 0; i < NLOADS; i++) store_unit(lds, regs, i);
  }
};

// ── operand contiguous along its row axis (M or N): thread -> (8-wide row chunk,
// group of 4 k) ; 4 loads of 16 bytes give a 4(k) x 8(row) block that is
// transposed in registers into 8 rows x 4 k and written as 8-byte LDS stores.
// When the tile has fewer 4x8 blocks than the workgroup has threads, the upper
// threads sit the staging out. ──
template <int ROWS>
struct PolyXC {
  static constexpr int CHUNKS = ROWS / 8;                 // row chunks per tile
  static constexpr int TOTAL = CHUNKS * (POLY_BK / 4);    // 4x8 blocks per tile
  static constexpr int NBLK = (TOTAL + POLY_NTHREADS - 1) / POLY_NTHREADS;
  static constexpr int NLOADS = NBLK * 4;
  // staging units for spreading the work over the K loop: unit u writes row pair u % 4 of
  // block u / 4; the four loads of a block can be reissued once its last unit is stored
  static constexpr int UNITS = NBLK * 4;
  static __device__ __forceinline__ bool active(int b) {
    return TOTAL % POLY_NTHREADS == 0 || (int)threadIdx.x + b * POLY_NTHREADS < TOTAL;
  }
  static __device__ __forceinline__ void load_block(const POLY_TIN *__restrict__ base, const int *chunk_off, const int *k_off,
                                                    poly_u32x4 (&regs)[NLOADS], int b) {
    if (active(b)) {
#pragma unroll
      for (int i = 0; i < 4; i++) regs[b * 4 + i] = *(const poly_u32x4_u *)(base + chunk_off[b] + k_off[b * 4 + i]);
    }
  }
  static __device__ __forceinline__ void store_unit(POLY_TIN *lds, const poly_u32x4 (&regs)[NLOADS], int u) {
    const int b = u >> 2, j = u & 3;
    if (!active(b)) return;
    const int c = threadIdx.x + b * POLY_NTHREADS;
    const int chunk = c % CHUNKS, kq = c / CHUNKS;
    // dword j of load i holds rows 2j (low half) and 2j+1 (high half) at k = kq*4+i
    const unsigned int a0 = regs[b * 4 + 0][j], a1 = regs[b * 4 + 1][j], a2 = regs[b * 4 + 2][j], a3 = regs[b * 4 + 3][j];
    poly_u32x2 lo, hi;
    lo[0] = (a0 & 0xffffu) | (a1 << 16);
    lo[1] = (a2 & 0xffffu) | (a3 << 16);
    hi[0] = (a0 >> 16) | (a1 & 0xffff0000u);
    hi[1] = (a2 >> 16) | (a3 & 0xffff0000u);
    const int r0 = chunk * 8 + 2 * j, r1 = r0 + 1;
    *(poly_u32x2 *)(lds + r0 * POLY_LDK + (((kq >> 1) ^ poly_swz(r0)) * 8) + (kq & 1) * 4) = lo;
    *(poly_u32x2 *)(lds + r1 * POLY_LDK + (((kq >> 1) ^ poly_swz(r1)) * 8) + (kq & 1) * 4) = hi;
  }
  static __device__ __forceinline__ void load(const POLY_TIN *__restrict__ base, const int *chunk_off, const int *k_off,
                                              poly_u32x4 (&regs)[NLOADS]) {
#pragma unroll
    for (int b = 0; b < NBLK; b++) load_block(base, chunk_off, k_off, regs, b);
  }
  static __device__ __forceinline__ void store(POLY_TIN *lds, const poly_u32x4 (&regs)[NLOADS]) {
#pragma unroll
    for (int u = 0; u < UNITS; u++) store_unit(lds, regs, u);
  }
};

extern "C" __global__ void __launch_bounds__(POLY_NTHREADS) poly_k(POLY_SIGNATURE) {
  // one allocation: the operand tiles during the K loop, the per-wave output staging after it
  __shared__ __attribute__((aligned(16))) POLY_TIN lds_raw[2 * (POLY_BM + POLY_BN) * POLY_LDK];
#ifdef POLY_EP_WIN_BYTES
  // The entries of the epilogue's lookup tables that most values hit.  Their loads are the
  // first the kernel issues; they go to LDS once the loads of the first operand tiles are
  // on their way (nothing waits for them alone), and the barriers of the K loop lie
  // between that and the epilogue's reads.
  __shared__ __attribute__((aligned(16))) unsigned char poly_win_raw[POLY_EP_WIN_BYTES];
  constexpr int WIN_VECS = (POLY_EP_WIN_BYTES / 16 + POLY_NTHREADS - 1) / POLY_NTHREADS;
  poly_u32x4 win_regs[WIN_VECS];
#pragma unroll
  for (int v = 0; v < WIN_VECS; v++) {
    const int b = ((int)threadIdx.x + v * POLY_NTHREADS) * 16;
    if (POLY_EP_WIN_BYTES / 16 % POLY_NTHREADS == 0 || b < POLY_EP_WIN_BYTES) win_regs[v] = *(const poly_u32x4 *)POLY_EP_WIN_SRC(b);
  }
  auto win_store = [&]() {
#pragma unroll
    for (int v = 0; v < WIN_VECS; v++) {
      const int b = ((int)threadIdx.x + v * POLY_NTHREADS) * 16;
      if (POLY_EP_WIN_BYTES / 16 % POLY_NTHREADS == 0 || b < POLY_EP_WIN_BYTES) *(poly_u32x4 *)(poly_win_raw + b) = win_regs[v];
    }
  };
#else
  auto win_store = [&]() {};
#endif
  auto lds_a = [&](int buf) { return lds_raw + buf * (POLY_BM * POLY_LDK); };
  auto lds_b = [&](int buf) { return lds_raw + 2 * POLY_BM * POLY_LDK + buf * (POLY_BN * POLY_LDK); };

  // Tile coordinates.  Consecutive workgroup ids go to different XCDs (8 of them,
  // each with its own L2), so ids are regrouped: all ids congruent mod 8 form one
  // contiguous run of tiles, and runs walk down M within a band of columns so the
  // B panel stays resident in that XCD's L2.
  constexpr int TILES_M = (POLY_M + POLY_BM - 1) / POLY_BM;
  constexpr int TILES_N = (POLY_N_HI - POLY_N_LO + POLY_BN - 1) / POLY_BN;
  constexpr int NT = TILES_M * TILES_N;
  int bid = blockIdx.x;
  {
    constexpr int PER = NT / 8, REM = NT % 8;
    const int xcd = bid & 7, idx = bid >> 3;
    bid = (xcd < REM ? xcd * (PER + 1) : REM * (PER + 1) + (xcd - REM) * PER) + idx;
  }
  // Within a run, tiles are visited in bands of POLY_GROUP_M tile rows (walking along N
  // inside a band) so that the workgroups resident on one XCD at a time share both A and
  // B panels.  When B is the larger operand the roles swap (POLY_GROUP_ALONG_N): bands of
  // tile columns, so that an XCD streams its slice of B once instead of all of B.
  int tile_m, tile_n;
  {
    constexpr int GM = POLY_GROUP_M;
#if POLY_GROUP_ALONG_N
    const int per_group = GM * TILES_M;
    const int group = bid / per_group, first_n = group * GM;
    const int gsz = (TILES_N - first_n) < GM ? (TILES_N - first_n) : GM;
    const int in_group = bid - group * per_group;
    tile_n = first_n + in_group % gsz;
    tile_m = in_group / gsz;
#else
    const int per_group = GM * TILES_N;
    const int group = bid / per_group, first_m = group * GM;
    const int gsz = (TILES_M - first_m) < GM ? (TILES_M - first_m) : GM;
    const int in_group = bid - group * per_group;
    tile_m = first_m + in_group % gsz;
    tile_n = in_group / gsz;
#endif
  }
#if POLY_KSPLIT > 1
  const int z = blockIdx.y / POLY_KSPLIT, poly_ks = blockIdx.y % POLY_KSPLIT;
  const int k_base = poly_ks * (POLY_KT * POLY_BK);
#else
  const int z = blockIdx.y;
  constexpr int k_base = 0;
#endif
  const int m0 = tile_m * POLY_BM, n0 = POLY_N_LO + tile_n * POLY_BN;

  const POLY_TIN *__restrict__ gA = POLY_A_PTR + poly_a_z(z);
  const POLY_TIN *__restrict__ gB = POLY_B_PTR + poly_b_z(z);

  // Per-thread global offsets of the rows (or row chunks) this thread stages.
  // Rows past the edge are clamped to the last valid row: they are loaded and
  // multiplied but never stored.
#if POLY_A_KC
  poly_u32x4 ra0[POLY_A_LOADS], ra1[POLY_A_LOADS];
  int a_off[POLY_A_LOADS];
#pragma unroll
  for (int i = 0; i < POLY_A_LOADS; i++) {
    int row = m0 + (threadIdx.x + i * POLY_NTHREADS) / (POLY_BK / 8);
    a_off[i] = poly_a_row(row < POLY_M ? row : POLY_M - 1);
  }
  typedef PolyKC<POLY_BM, POLY_A_LOADS> StageA;
#else
  typedef PolyXC<POLY_BM> StageA;
  poly_u32x4 ra0[StageA::NLOADS], ra1[StageA::NLOADS];
  int a_off[StageA::NBLK], a_kq[StageA::NBLK];
#pragma unroll
  for (int b = 0; b < StageA::NBLK; b++) {
    const int c = (threadIdx.x + b * POLY_NTHREADS) % StageA::TOTAL;
    int row = m0 + (c % (POLY_BM / 8)) * 8;
    a_off[b] = poly_a_row(row < POLY_M ? row : POLY_M - 8);
    a_kq[b] = (c / (POLY_BM / 8)) * 4;
  }
#endif
#if POLY_B_KC
  poly_u32x4 rb0[POLY_B_LOADS], rb1[POLY_B_LOADS];
  int b_off[POLY_B_LOADS];
#pragma unroll
  for (int i = 0; i < POLY_B_LOADS; i++) {
    int row = n0 + (threadIdx.x + i * POLY_NTHREADS) / (POLY_BK / 8);
    b_off[i] = poly_b_row(row < POLY_N ? row : POLY_N - 1);
  }
  typedef PolyKC<POLY_BN, POLY_B_LOADS> StageB;
#else
  typedef PolyXC<POLY_BN> StageB;
  poly_u32x4 rb0[StageB::NLOADS], rb1[StageB::NLOADS];
  int b_off[StageB::NBLK], b_kq[StageB::NBLK];
#pragma unroll
  for (int b = 0; b < StageB::NBLK; b++) {
    const int c = (threadIdx.x + b * POLY_NTHREADS) % StageB::TOTAL;
    int row = n0 + (c % (POLY_BN / 8)) * 8;
    b_off[b] = poly_b_row(row < POLY_N ? row : POLY_N - 8);
    b_kq[b] = (c / (POLY_BN / 8)) * 4;
  }
#endif

  auto load_tiles = [&](int kt, auto &ra, auto &rb) {
    const int k0 = k_base + kt * POLY_BK;
#if POLY_A_KC
    StageA::load(gA, a_off, poly_a_k(k0), ra);
#else
    int ak[StageA::NLOADS];
#pragma unroll
    for (int b = 0; b < StageA::NBLK; b++)
#pragma unroll
      for (int i = 0; i < 4; i++) ak[b * 4 + i] = poly_a_k(k0 + a_kq[b] + i);
    StageA::load(gA, a_off, ak, ra);
#endif
#if POLY_B_KC
    StageB::load(gB, b_off, poly_b_k(k0), rb);
#else
    int bk[StageB::NLOADS];
#pragma unroll
    for (int b = 0; b < StageB::NBLK; b++)
#pragma unroll
      for (int i = 0; i < 4; i++) bk[b * 4 + i] = poly_b_k(k0 + b_kq[b] + i);
    StageB::load(gB, b_off, bk, rb);
#endif
  };

  // One piece of the staging work, for spreading it between the MFMAs of the K loop:
  // the units of both operands that fall into part `part` of `nparts` write their share
  // of the tile held in (ra, rb) to LDS buffer `buf` (if st) and then refill those
  // registers from tile kt_load (if ld).
  auto stage_part = [&](int part, int nparts, bool st, int buf, bool ld, int kt_load, auto &ra, auto &rb) {
    const int k0 = k_base + kt_load * POLY_BK;
#pragma unroll
    for (int u = 0; u < StageA::UNITS; u++) {
      if (u * nparts / StageA::UNITS != part) continue;
      if (st) StageA::store_unit(lds_a(buf), ra, u);
#if POLY_A_KC
      if (ld) StageA::load_unit(gA, a_off, poly_a_k(k0), ra, u);
#else
      if (ld && (u & 3) == 3) {
        int ak[StageA::NLOADS];
#pragma unroll
        for (int i = 0; i < 4; i++) ak[(u >> 2) * 4 + i] = poly_a_k(k0 + a_kq[u >> 2] + i);
        StageA::load_block(gA, a_off, ak, ra, u >> 2);
      }
#endif
    }
#pragma unroll
    for (int u = 0; u < StageB::UNITS; u++) {
      if (u * nparts / StageB::UNITS != part) continue;
      if (st) StageB::store_unit(lds_b(buf), rb, u);
#if POLY_B_KC
      if (ld) StageB::load_unit(gB, b_off, poly_b_k(k0), rb, u);
#else
      if (ld && (u & 3) == 3) {
        int bk[StageB::NLOADS];
#pragma unroll
        for (int i = 0; i < 4; i++) bk[(u >> 2) * 4 + i] = poly_b_k(k0 + b_kq[u >> 2] + i);
        StageB::load_block(gB, b_off, bk, rb, u >> 2);
      }
#endif
    }
  };

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave % POLY_WAVES_M) * POLY_WM, wn = (wave / POLY_WAVES_M) * POLY_WN;
  const int frag_row = lane & 31;

  poly_acc16 acc[POLY_TM][POLY_TN];
#pragma unroll
  for (int i = 0; i < POLY_TM; i++)
#pragma unroll
    for (int j = 0; j < POLY_TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  // fragment addresses: row part and per-tile swizzle are loop invariant
  int a_row_off[POLY_TM], a_swz[POLY_TM], b_row_off[POLY_TN], b_swz[POLY_TN];
#pragma unroll
  for (int i = 0; i < POLY_TM; i++) { const int r = wm + i * 32 + frag_row; a_row_off[i] = r * POLY_LDK; a_swz[i] = poly_swz(r); }
#pragma unroll
  for (int j = 0; j < POLY_TN; j++) { const int r = wn + j * 32 + frag_row; b_row_off[j] = r * POLY_LDK; b_swz[j] = poly_swz(r); }
  const int frag_col = lane >> 5;   // which 8-wide half of a 16-deep K step

  // Fragment registers.  Small wave tiles keep two sets (the reads of K step ks+1 are
  // issued before the MFMAs of step ks).  Wave tiles of 8 or more MFMAs per step keep one
  // set and refill it on the fly: MFMAs run row by row, so the A fragment of row i is
  // dead after its last column and the B fragment of column j after the last row; each is
  // reread for the next step right there, at least three MFMAs before its next use.
#ifndef POLY_FRAG_ROLL
#define POLY_FRAG_ROLL (POLY_TM * POLY_TN >= 8)
#endif
  poly_in8 fa[POLY_FRAG_ROLL ? 1 : 2][POLY_TM], fb[POLY_FRAG_ROLL ? 1 : 2][POLY_TN];
  auto read_a = [&](int cur, int ks, int buf, int i) {
    fa[buf][i] = *(const poly_in8 *)(lds_a(cur) + a_row_off[i] + (((ks * 2 + frag_col) ^ a_swz[i]) * 8));
  };
  auto read_b = [&](int cur, int ks, int buf, int j) {
    fb[buf][j] = *(const poly_in8 *)(lds_b(cur) + b_row_off[j] + (((ks * 2 + frag_col) ^ b_swz[j]) * 8));
  };
  auto read_frags = [&](int cur, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < POLY_TM; i++) read_a(cur, ks, buf, i);
#pragma unroll
    for (int j = 0; j < POLY_TN; j++) read_b(cur, ks, buf, j);
  };

  // The K loop keeps the matrix pipe and the LDS pipe busy at the same time.  A K tile is
  // KS steps of MT MFMAs: KS * MT slots.  Each slot issues one MFMA, then the fragment
  // refills that became possible, then its share of the staging work (LDS stores of the
  // next tile, global loads of a later one), so that the stores drain while the MFMAs
  // execute instead of in a phase of their own.  The order is pinned slot by slot.
  constexpr int KS = POLY_BK / 16, MT = POLY_TM * POLY_TN;
  auto k_tile = [&](int cur, auto &&stage_slot) {
    read_frags(cur, 0, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      constexpr int R = POLY_FRAG_ROLL;
      if (!R && ks + 1 < KS) read_frags(cur, ks + 1, (ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < POLY_TM; i++)
#pragma unroll
        for (int j = 0; j < POLY_TN; j++) {
          const int buf = R ? 0 : (ks & 1);
          acc[i][j] = POLY_MFMA(fa[buf][i], fb[buf][j], acc[i][j]);
          if (R && ks + 1 < KS) {
            if (j == POLY_TN - 1) read_a(cur, ks + 1, 0, i);
            if (i == POLY_TM - 1) read_b(cur, ks + 1, 0, j);
          }
          stage_slot(ks * MT + i * POLY_TN + j);
          // (small wave tiles: pinned per K step only, the compiler places the staging
          // work among the step's few MFMAs)
          if (R) __builtin_amdgcn_sched_barrier(0);
        }
      if (!R) __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };

#if POLY_PIPE == 3
  // Three tiles deep: tile kt is multiplied out of one LDS buffer; tile kt+1 waits in
  // one register set and moves to the other LDS buffer during the iteration; tile kt+2
  // is in flight into the second register set; each register of the first set is
  // refilled from tile kt+3 as soon as it is stored.  Every global load has about two
  // iterations to land.  Tile t always uses register set t & 1, hence the loop is
  // unrolled by two.
  load_tiles(0, ra0, rb0);
  win_store();
  StageA::store(lds_a(0), ra0);
  StageB::store(lds_b(0), rb0);
  if (POLY_KT > 1) load_tiles(1, ra1, rb1);
  if (POLY_KT > 2) load_tiles(2, ra0, rb0);
  __syncthreads();

  auto iteration = [&](int kt, auto &ra_next, auto &rb_next, bool st, bool ld) {
    const int cur = kt & 1;
    k_tile(cur, [&](int slot) { stage_part(slot, KS * MT, st, cur ^ 1, ld, kt + 3, ra_next, rb_next); });
  };
  // steady state (every iteration stores and loads: no branches in the loop body), then
  // the last iterations with their conditions known at compile time
  constexpr int STEADY = POLY_KT >= 3 ? ((POLY_KT - 3) & ~1) : 0;
  for (int kt = 0; kt < STEADY; kt += 2) {
    iteration(kt, ra1, rb1, true, true);
    iteration(kt + 1, ra0, rb0, true, true);
  }
#pragma unroll
  for (int kt = STEADY; kt < POLY_KT; kt++) {
    if (kt & 1) iteration(kt, ra0, rb0, kt + 1 < POLY_KT, kt + 3 < POLY_KT);
    else iteration(kt, ra1, rb1, kt + 1 < POLY_KT, kt + 3 < POLY_KT);
  }
#else
  // Two tiles deep (for tiles whose accumulators leave no room for a second staging
  // register set): the global loads of tile kt+1 are issued at the top of iteration kt
  // and move to the other LDS buffer during the second half of its slots.
  load_tiles(0, ra0, rb0);
  win_store();
  StageA::store(lds_a(0), ra0);
  StageB::store(lds_b(0), rb0);
  __syncthreads();
  auto iteration = [&](int kt, bool st) {
    const int cur = kt & 1;
    if (st) load_tiles(kt + 1, ra0, rb0);
    constexpr int FIRST = (KS / 2) * MT, NSLOTS = KS * MT - FIRST;
    k_tile(cur, [&](int slot) {
      if (slot >= FIRST) stage_part(slot - FIRST, NSLOTS, st, cur ^ 1, false, 0, ra0, rb0);
    });
  };
  for (int kt = 0; kt + 1 < POLY_KT; kt++) iteration(kt, true);
  iteration(POLY_KT - 1, false);
#endif

  // Accumulator layout of the 32x32 MFMA: register r of lane l holds
  // row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the tile: a lane owns one column, so
  // its stores would be single elements.  Each 32x32 tile therefore goes through a
  // per-wave LDS staging area and comes back with 8 consecutive columns of one row per
  // lane, so that whatever the epilogue loads and stores along n is 16 bytes wide (for
  // 16-bit data) and a wave writes full 64-byte row segments.
#if !POLY_EP_CONTIG && POLY_N % 8 != 0
  // Neither rows of 8 nor contiguous: store straight from the accumulator layout, where
  // the 32 lanes of a half-wave write 32 consecutive columns.
#pragma unroll
  for (int i = 0; i < POLY_TM; i++)
#pragma unroll
    for (int j = 0; j < POLY_TN; j++) {
      const int n = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int m = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < POLY_M && n < POLY_N) { POLY_EPILOGUE(acc[i][j][r], m, n, z); }
      }
    }
#else
  static_assert(POLY_NTHREADS / 64 * 32 * POLY_STAGE_LD * 4 <= (int)sizeof(lds_raw), "staging area exceeds the operand tiles");
  __syncthreads();   // every wave is done reading the operand tiles
  float *const stage = (float *)lds_raw + wave * (32 * POLY_STAGE_LD);
#pragma unroll
  for (int i = 0; i < POLY_TM; i++)
#pragma unroll
    for (int j = 0; j < POLY_TN; j++) {
#pragma unroll
      for (int r = 0; r < 16; r++)
        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * POLY_STAGE_LD + (lane & 31)] = acc[i][j][r];
      // LDS operations of one wave complete in order; the fences only keep the compiler
      // from moving the reads above the writes (and the next tile's writes above the reads)
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int row = (lane >> 2) + 16 * h, c0 = (lane & 3) * 8;
        const poly_f32x4 lo = *(const poly_f32x4 *)(stage + row * POLY_STAGE_LD + c0);
        const poly_f32x4 hi = *(const poly_f32x4 *)(stage + row * POLY_STAGE_LD + c0 + 4);
        const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const int m = m0 + wm + i * 32 + row, n = n0 + wn + j * 32 + c0;
#if POLY_EP_CONTIG
        if (m < POLY_M && n < POLY_N) {
          // 8 finished values of one row; a full group goes out as one store (rows need
          // not start on 16-byte boundaries: global stores take any alignment)
          typedef POLY_EP_TYPE poly_out8 __attribute__((ext_vector_type(8)));
          typedef poly_out8 poly_out8_u __attribute__((aligned(sizeof(POLY_EP_TYPE))));
          poly_out8 o;
#if defined(POLY_EP_WIN_BYTES) && defined(POLY_EP_VALUE_WIN)
          // table lookups from the LDS windows first; a lane with an input outside them
          // computes its group again with lookups in memory
          unsigned int poly_tmax = 0;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const int ne = (POLY_N % 8 == 0 || n + e < POLY_N) ? n + e : n;
            o[e] = POLY_EP_VALUE_WIN(v[e], m, ne, z);
          }
          if (poly_tmax >= POLY_WIN_CODES)
#endif
#pragma unroll
          for (int e = 0; e < 8; e++) {
            // (keep n + e plain when every group is full: whatever the epilogue loads
            // along n must stay visibly consecutive to be fetched as one vector)
            const int ne = (POLY_N % 8 == 0 || n + e < POLY_N) ? n + e : n;
            o[e] = POLY_EP_VALUE(v[e], m, ne, z);
          }
          if (POLY_N % 8 == 0 || n + 7 < POLY_N) {
            *(poly_out8_u *)POLY_EP_PTR(m, n, z) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
              if (n + e < POLY_N) *POLY_EP_PTR(m, n + e, z) = o[e];
          }
#ifdef POLY_EP_MID_VALUE
          {
            // a value on the way to the stored one that other kernels read as well: stored too
            typedef POLY_EP_MID_TYPE poly_mid8 __attribute__((ext_vector_type(8)));
            typedef poly_mid8 poly_mid8_u __attribute__((aligned(sizeof(POLY_EP_MID_TYPE))));
            poly_mid8 mv;
#pragma unroll
            for (int e = 0; e < 8; e++) {
              const int ne = (POLY_N % 8 == 0 || n + e < POLY_N) ? n + e : n;
              mv[e] = POLY_EP_MID_VALUE(v[e], m, ne, z);
            }
            if (POLY_N % 8 == 0 || n + 7 < POLY_N) {
              *(poly_mid8_u *)POLY_EP_MID_PTR(m, n, z) = mv;
            } else {
#pragma unroll
              for (int e = 0; e < 8; e++)
                if (n + e < POLY_N) *POLY_EP_MID_PTR(m, n + e, z) = mv[e];
            }
          }
#endif
        }
#else
        if (m < POLY_M && n < POLY_N) {
#pragma unroll
          for (int e = 0; e < 8; e++) { POLY_EPILOGUE(v[e], m, n + e, z); }
        }
#endif
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
#endif
}
