// matmul_dma.hip -- hand-written CDNA4 (gfx950) matmul template whose operand tiles go
// from global memory straight into LDS (global_load_lds_dwordx4), without passing
// through registers.
//
// C[z][m][n] = epilogue( sum_k A(z,m,k) * B(z,k,n) ) with 16-bit float inputs (bf16 or
// fp16) and fp32 accumulation on the 32x32x16 MFMA.  The renderer (templates.cc)
// instantiates it by prepending the same configuration block as for matmul_mfma.hip
// (POLY_TIN, POLY_MFMA, POLY_M/N/K/Z, POLY_BM/BN/BK, POLY_WAVES_M/N, POLY_A_KC/B_KC,
// POLY_A_PTR/B_PTR, poly_a_row/poly_b_row/poly_a_z/poly_b_z/poly_a_k/poly_b_k,
// POLY_SIGNATURE, the POLY_EP* epilogue macros, POLY_KSPLIT, POLY_N_LO/HI, POLY_GROUP_M,
// POLY_GROUP_ALONG_N) plus
//
//   POLY_STAGES         LDS stages of one K tile (POLY_BK deep) each; loads run
//                       POLY_STAGES - 1 tiles ahead of the multiplication
//   POLY_WG_PER_CU      workgroups meant to share a CU (sets the register budget), so
//                       that one's epilogue runs under another's K loop
//   POLY_TOUCH_WGS      (optional) that many extra workgroups at the front of the grid, which
//                       multiply nothing: they read one word of every 64 bytes of the
//                       POLY_TOUCH_LINES * 64 bytes from element POLY_TOUCH_FIRST of B on and
//                       leave.  When B comes from HBM (weights), they run ahead of the others
//                       through B, which then find it in the memory-side cache instead of
//                       waiting for HBM at every K tile
//   POLY_EP_WIN_BYTES   (optional, set by the epilogue's own code when POLY_EP_WIN_ROOM
//                       suffices) bytes of the epilogue's lookup tables that the kernel
//                       keeps in LDS, read from POLY_EP_WIN_SRC(byte): they are loaded
//                       into the first stage that the K loop no longer needs, during its
//                       last iterations, so the window costs no LDS of its own
//
//   POLY_EP_MID_TYPE, POLY_EP_MID_VALUE(acc, m, n, z), POLY_EP_MID_PTR(m, n, z)
//                       (optional, with POLY_EP_CONTIG) a second output with the layout of the
//                       first: a value the epilogue passes through on its way, stored as well
//   POLY_EP_BLOCKMAX_LO, POLY_EP_BLOCKMAX_HI, POLY_EP_BLOCKMAX_IDX(m, n), POLY_EP_BLOCKMAX_PTR
//                       (optional, with POLY_EP_CONTIG and tiles of whole 64 x 64 blocks)
//                       the columns [LO, HI) of the output, both multiples of 64, are read
//                       by a later launch in blocks of 64 rows x 64 columns that wants a
//                       bound on the magnitudes in each: the largest |stored value| of the
//                       block whose first element is (m, n) goes, as the bits of the float,
//                       to POLY_EP_BLOCKMAX_PTR[POLY_EP_BLOCKMAX_IDX(m, n)] (a NaN counts
//                       as larger than everything).  Every block lies inside one
//                       workgroup's tile: plain stores, nothing to clear beforehand
//
// Data path.  One global_load_lds_dwordx4 moves 16 bytes per lane from any global
// address to LDS address M0 + 16 * lane: a wave fills 1024 consecutive bytes of LDS per
// instruction, and which global chunk lands in which 16-byte slot is the lane's choice
// of source address.  The tiles keep the layouts the fragment reads want:
//   operand contiguous along K:  LDS [row][BK], the 16-byte columns of a row XOR-swizzled
//       by the row number; fragments are 16-byte reads (8 consecutive k of one row);
//   operand contiguous along its row axis (M or N):  LDS [k][rows], the 16-byte chunks of
//       a k-row XOR-swizzled by k; fragments are two ds_read_b64_tr_b16 (a 4 x 16 block
//       comes back transposed: lane j of a group of 16 holds 4 consecutive k of row j).
// Completion of the loads is counted by hand (s_waitcnt vmcnt) before the barrier that
// opens a stage: the compiler does not see these loads, and inside the K loop there are
// no other vector memory operations, so the counter holds exactly the LDS loads issued.
#ifdef POLY_TEMPLATE_STANDALONE
#include <hip/hip_runtime.h>
#define POLY_TIN __bf16
#define POLY_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)
#define POLY_M 4096
#define POLY_N 4096
#define POLY_K 4096
#define POLY_Z 1
#define POLY_BM 256
#define POLY_BN 128
#define POLY_BK 32
#define POLY_STAGES 3
#define POLY_WG_PER_CU 2
#define POLY_GROUP_M 8
#define POLY_GROUP_ALONG_N 0
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
typedef float poly_acc16 __attribute__((ext_vector_type(16)));
typedef unsigned int poly_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int poly_u32x2 __attribute__((ext_vector_type(2)));
typedef short poly_s16x4 __attribute__((ext_vector_type(4)));
typedef float poly_f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) poly_s16x4 poly_lds_s16x4;

#define POLY_NW (POLY_WAVES_M * POLY_WAVES_N)
#define POLY_NTHREADS (64 * POLY_NW)
#define POLY_WM (POLY_BM / POLY_WAVES_M)
#define POLY_WN (POLY_BN / POLY_WAVES_N)
#define POLY_TM (POLY_WM / 32)
#define POLY_TN (POLY_WN / 32)
#ifndef POLY_KSPLIT
#define POLY_KSPLIT 1
#endif
#ifndef POLY_N_LO
#define POLY_N_LO 0
#define POLY_N_HI POLY_N
#endif
#ifndef POLY_KT
#define POLY_KT (POLY_K / POLY_BK / POLY_KSPLIT)
#endif
#ifndef POLY_WG_PER_CU
#define POLY_WG_PER_CU 1
#endif
#define POLY_STAGE_LD 36

// bytes of one operand tile, LDS-load instructions (1024 bytes each) per tile and per wave
#define POLY_A_BYTES (POLY_BM * POLY_BK * 2)
#define POLY_B_BYTES (POLY_BN * POLY_BK * 2)
#define POLY_STAGE_BYTES (POLY_A_BYTES + POLY_B_BYTES)
#define POLY_A_NI (POLY_A_BYTES / 1024)
#define POLY_B_NI (POLY_B_BYTES / 1024)
#define POLY_A_IPW (POLY_A_NI / POLY_NW)
#define POLY_B_IPW (POLY_B_NI / POLY_NW)
#define POLY_IPW (POLY_A_IPW + POLY_B_IPW)
static_assert(POLY_A_NI % POLY_NW == 0 && POLY_B_NI % POLY_NW == 0, "every wave issues the same number of LDS loads per tile");
static_assert(POLY_BK == 32 || POLY_BK == 64, "K tile of 32 or 64");

// ── layouts ────────────────────────────────────────────────────────────────
// K-contiguous operand, [row][BK]: BK/8 chunks of 16 bytes per row.  A 16-byte fragment
// read is served 16 lanes at a time over 256 bytes of banks: the 16 lanes read the same
// logical chunk of 16 consecutive rows, which must land on 16 different 16-byte slots
// modulo 256 bytes.  With 8 chunks (rows of 128 bytes, two rows per 256) the chunk index
// is XORed with the row number and with the row number / 8; with 4 chunks (rows of 64
// bytes, four rows per 256) with the row number / 4.
#define POLY_CH (POLY_BK / 8)
__device__ __forceinline__ int poly_swz_k(int row) { return POLY_CH == 8 ? ((row ^ (row >> 3)) & 7) : ((row >> 2) & 3); }
// Row-contiguous operand, [k][ROWS]: a transposing read is served 32 lanes at a time, which
// touch 4 consecutive k-rows x 64 bytes (the same four logical chunks of each), 256 bytes in
// all: the four k-rows have to land on the four different 64-byte groups of banks.  A k-row is
// a multiple of 256 bytes long when ROWS is a multiple of 128, so without a swizzle they all
// land on one; the chunk index is XORed with (k mod 4) * 4, which moves k-row k by k mod 4
// groups.  (Other row counts -- 64, 192 -- keep a swizzle inside blocks of 8 chunks, which
// pairs the four k-rows on two groups.)
template <int ROWS>
__device__ __forceinline__ int poly_swz_x(int k) { return (ROWS % 128 == 0) ? ((k & 3) << 2) : ((k & 3) | ((k & 1) << 2)); }

// One LDS load: 16 bytes per lane from `base + voff` to LDS byte address lds_addr + 16 * lane.
#ifdef POLY_HOST_ADDRESS_CHECK   // the kernel compiled for the host to check its indexing: lanes run one by one, LDS addresses count from the array
static unsigned char *poly_host_lds;
__device__ __forceinline__ void poly_lds_load(unsigned lds_addr, unsigned voff, const void *base) {
  memcpy(poly_host_lds + lds_addr + 16 * (threadIdx.x & 63), (const unsigned char *)base + voff, 16);
}
__device__ __forceinline__ void poly_lds_load_flat(unsigned lds_addr, const void *src) { memcpy(poly_host_lds + lds_addr + 16 * (threadIdx.x & 63), src, 16); }
__device__ __forceinline__ void poly_wait_vm(int) {}
#define __builtin_amdgcn_s_barrier() ((void)0)
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) (*(p))
#else
__device__ __forceinline__ void poly_lds_load(unsigned lds_addr, unsigned voff, const void *base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
// (the same with a full address per lane)
__device__ __forceinline__ void poly_lds_load_flat(unsigned lds_addr, const void *src) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(src) : "memory", "m0");
}
// s_waitcnt vmcnt(n) for an n that constant propagation settles (the counter has 6 bits)
__device__ __forceinline__ void poly_wait_vm(int n) {
#define POLY_VM_CASE(i) case i: asm volatile("s_waitcnt vmcnt(" #i ")" ::: "memory"); break;
  switch (n) {
    POLY_VM_CASE(0) POLY_VM_CASE(1) POLY_VM_CASE(2) POLY_VM_CASE(3) POLY_VM_CASE(4) POLY_VM_CASE(5) POLY_VM_CASE(6) POLY_VM_CASE(7)
    POLY_VM_CASE(8) POLY_VM_CASE(9) POLY_VM_CASE(10) POLY_VM_CASE(11) POLY_VM_CASE(12) POLY_VM_CASE(13) POLY_VM_CASE(14) POLY_VM_CASE(15)
    POLY_VM_CASE(16) POLY_VM_CASE(17) POLY_VM_CASE(18) POLY_VM_CASE(19) POLY_VM_CASE(20) POLY_VM_CASE(21) POLY_VM_CASE(22) POLY_VM_CASE(23)
    POLY_VM_CASE(24) POLY_VM_CASE(25) POLY_VM_CASE(26) POLY_VM_CASE(27) POLY_VM_CASE(28) POLY_VM_CASE(29) POLY_VM_CASE(30) POLY_VM_CASE(31)
    POLY_VM_CASE(32) POLY_VM_CASE(33) POLY_VM_CASE(34) POLY_VM_CASE(35) POLY_VM_CASE(36) POLY_VM_CASE(37) POLY_VM_CASE(38) POLY_VM_CASE(39)
    POLY_VM_CASE(40) POLY_VM_CASE(41) POLY_VM_CASE(42) POLY_VM_CASE(43) POLY_VM_CASE(44) POLY_VM_CASE(45) POLY_VM_CASE(46) POLY_VM_CASE(47)
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
#undef POLY_VM_CASE
}
#endif

// (register budget: the waves of POLY_WG_PER_CU workgroups share a SIMD)
#if POLY_WG_PER_CU * POLY_NW > 4 && !defined(POLY_HOST_ADDRESS_CHECK)
#define POLY_WAVES_ATTR __attribute__((amdgpu_waves_per_eu(POLY_WG_PER_CU * POLY_NW / 4, POLY_WG_PER_CU * POLY_NW / 4)))
#else
#define POLY_WAVES_ATTR
#endif
extern "C" __global__ void __launch_bounds__(POLY_NTHREADS) POLY_WAVES_ATTR poly_k(POLY_SIGNATURE) {
  // one allocation: the operand stages during the K loop, the per-wave output staging after it
  __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[POLY_STAGES * POLY_STAGE_BYTES];
  constexpr int S = POLY_STAGES;
#ifdef POLY_EP_WIN_BYTES
  // The lookup-table window lives in the stage of tile KT - S, the first one the K loop
  // leaves for good; the output staging of the epilogue lies before or behind it.
  static_assert(POLY_KT >= S && S >= 2 && (POLY_EP_WIN_BYTES + 1023) / 1024 * 1024 <= POLY_STAGE_BYTES, "no stage for the window");
  constexpr int WIN_STAGE = (POLY_KT - S) % S;
  constexpr int WIN_NI = (POLY_EP_WIN_BYTES + 1023) / 1024, WIN_IPW = (WIN_NI + POLY_NW - 1) / POLY_NW;
  unsigned char *const poly_win_raw = lds_raw + WIN_STAGE * POLY_STAGE_BYTES;
  constexpr int OUT_BYTES = POLY_NW * 32 * POLY_STAGE_LD * 4;
  constexpr int OUT_OFF = OUT_BYTES <= WIN_STAGE * POLY_STAGE_BYTES ? 0 : (WIN_STAGE + 1) * POLY_STAGE_BYTES;
  static_assert(OUT_OFF + OUT_BYTES <= S * POLY_STAGE_BYTES, "no room for the output staging beside the window");
#else
  constexpr int OUT_OFF = 0, WIN_IPW = 0;
  static_assert(POLY_NW * 32 * POLY_STAGE_LD * 4 <= S * POLY_STAGE_BYTES, "staging area exceeds the operand stages");
#endif

  // Tile coordinates: ids congruent mod 8 (one XCD, one L2) form a contiguous run of
  // tiles; within a run, bands of POLY_GROUP_M tile rows (or tile columns).
  constexpr int TILES_M = (POLY_M + POLY_BM - 1) / POLY_BM;
  constexpr int TILES_N = (POLY_N_HI - POLY_N_LO + POLY_BN - 1) / POLY_BN;
  constexpr int NT = TILES_M * TILES_N;
#ifdef POLY_TOUCH_WGS
  static_assert(POLY_TOUCH_WGS % 8 == 0, "the workgroups behind keep their XCDs");
  if (blockIdx.x < POLY_TOUCH_WGS) {
    if (blockIdx.y == 0) {
      const unsigned int *const p = (const unsigned int *)(POLY_B_PTR + (POLY_TOUCH_FIRST));
      unsigned int a = 0;
      for (long long i = (long long)blockIdx.x * POLY_NTHREADS + threadIdx.x; i < (POLY_TOUCH_LINES); i += (long long)POLY_TOUCH_WGS * POLY_NTHREADS) a ^= p[i * 16];
      asm volatile("" ::"v"(a));
    }
    return;
  }
  int bid = blockIdx.x - POLY_TOUCH_WGS;
#else
  int bid = blockIdx.x;
#endif
#ifdef POLY_EP_BLOCKMAX_LO
  static_assert(POLY_BM % 64 == 0 && POLY_BN % 64 == 0 && POLY_M % 64 == 0 && (POLY_EP_BLOCKMAX_LO) % 64 == 0 && (POLY_EP_BLOCKMAX_HI) % 64 == 0, "whole blocks per tile");
  constexpr int BLK_N = POLY_BN / 64, BLK_COUNT = (POLY_BM / 64) * BLK_N;
  __shared__ unsigned int poly_blk[BLK_COUNT];
  if (threadIdx.x < BLK_COUNT) poly_blk[threadIdx.x] = 0u;      // (published by the K loop's barriers)
#endif
  {
    constexpr int PER = NT / 8, REM = NT % 8;
    const int xcd = bid & 7, idx = bid >> 3;
    bid = (xcd < REM ? xcd * (PER + 1) : REM * (PER + 1) + (xcd - REM) * PER) + idx;
  }
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

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
#ifdef POLY_HOST_ADDRESS_CHECK
  const unsigned lds_base = 0;
  poly_host_lds = lds_raw;
#else
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)lds_raw;
#endif

  // ── per-lane source offsets of this wave's LDS loads ─────────────────────────
  // Wave w issues instructions q * NW + w (q = 0 .. IPW-1) of each operand tile;
  // instruction i fills bytes [1024 i, 1024 i + 1024) of the tile.  Rows past the edge
  // are clamped to the last valid row: loaded and multiplied, never stored.
  // K-contiguous: byte b of the tile is row b / (2 BK), physical chunk (b / 16) % CH.
  // Row-contiguous: byte b is k-row b / (2 ROWS), physical chunk (b / 16) % (ROWS / 8).
  int a_off[POLY_A_IPW], a_kin[POLY_A_IPW], b_off[POLY_B_IPW], b_kin[POLY_B_IPW];
#pragma unroll
  for (int q = 0; q < POLY_A_IPW; q++) {
    const int slot = (q * POLY_NW + wave) * 64 + lane;      // 16-byte slot of the tile
#if POLY_A_KC
    const int row = slot / POLY_CH, c = (slot % POLY_CH) ^ poly_swz_k(row);
    const int m = m0 + row;
    a_off[q] = poly_a_row(m < POLY_M ? m : POLY_M - 1) + c * 8;
    a_kin[q] = 0;
#else
    const int kin = slot / (POLY_BM / 8), c = (slot % (POLY_BM / 8)) ^ poly_swz_x<POLY_BM>(kin);
    const int m = m0 + c * 8;
    a_off[q] = poly_a_row(m < POLY_M ? m : POLY_M - 8);
    a_kin[q] = kin;
#endif
  }
#pragma unroll
  for (int q = 0; q < POLY_B_IPW; q++) {
    const int slot = (q * POLY_NW + wave) * 64 + lane;
#if POLY_B_KC
    const int row = slot / POLY_CH, c = (slot % POLY_CH) ^ poly_swz_k(row);
    const int n = n0 + row;
    b_off[q] = poly_b_row(n < POLY_N ? n : POLY_N - 1) + c * 8;
    b_kin[q] = 0;
#else
    const int kin = slot / (POLY_BN / 8), c = (slot % (POLY_BN / 8)) ^ poly_swz_x<POLY_BN>(kin);
    const int n = n0 + c * 8;
    b_off[q] = poly_b_row(n < POLY_N ? n : POLY_N - 8);
    b_kin[q] = kin;
#endif
  }
  // unit u of a tile's loads: A instructions first, then B
  auto issue_unit = [&](int u, int kt, int stage) {
    const int k0 = k_base + kt * POLY_BK;
    if (u < POLY_A_IPW) {
      const int q = u;
      const unsigned lds = lds_base + (unsigned)(stage * POLY_STAGE_BYTES + q * POLY_NW * 1024) + (unsigned)wave * 1024u;
      const int off = a_off[q] + poly_a_k(k0 + a_kin[q]);
      poly_lds_load(lds, (unsigned)off * 2u, gA);
    } else {
      const int q = u - POLY_A_IPW;
      const unsigned lds = lds_base + (unsigned)(stage * POLY_STAGE_BYTES + POLY_A_BYTES + q * POLY_NW * 1024) + (unsigned)wave * 1024u;
      const int off = b_off[q] + poly_b_k(k0 + b_kin[q]);
      poly_lds_load(lds, (unsigned)off * 2u, gB);
    }
  };
  auto issue_tile = [&](int kt, int stage) {
#pragma unroll
    for (int u = 0; u < POLY_IPW; u++) issue_unit(u, kt, stage);
  };

  const int wm = (wave % POLY_WAVES_M) * POLY_WM, wn = (wave / POLY_WAVES_M) * POLY_WN;

  poly_acc16 acc[POLY_TM][POLY_TN];
#pragma unroll
  for (int i = 0; i < POLY_TM; i++)
#pragma unroll
    for (int j = 0; j < POLY_TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  // ── fragment addresses (bytes within an operand tile), loop invariant ────────
  // K-contiguous: lane reads 16 bytes of row (l % 32) at chunk 2 ks + l / 32.
  // Row-contiguous: lane l of a transposing read points at k = 8 (l / 32) + (l % 16) / 4
  // (+ 16 ks + 4 t) and at rows x0 + 16 ((l / 16) % 2) + 4 (l % 4) .. + 3.
  int a_fr[POLY_TM], a_sw[POLY_TM], b_fr[POLY_TN], b_sw[POLY_TN];
#pragma unroll
  for (int i = 0; i < POLY_TM; i++) {
#if POLY_A_KC
    const int r = wm + i * 32 + (lane & 31);
    a_fr[i] = r * (POLY_BK * 2); a_sw[i] = poly_swz_k(r);
#else
    const int kl = 8 * (lane >> 5) + ((lane & 15) >> 2), x = wm + i * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    a_fr[i] = kl * (POLY_BM * 2) + (((x >> 3) ^ poly_swz_x<POLY_BM>(kl)) * 16) + (x & 7) * 2; a_sw[i] = 0;
#endif
  }
#pragma unroll
  for (int j = 0; j < POLY_TN; j++) {
#if POLY_B_KC
    const int r = wn + j * 32 + (lane & 31);
    b_fr[j] = r * (POLY_BK * 2); b_sw[j] = poly_swz_k(r);
#else
    const int kl = 8 * (lane >> 5) + ((lane & 15) >> 2), x = wn + j * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    b_fr[j] = kl * (POLY_BN * 2) + (((x >> 3) ^ poly_swz_x<POLY_BN>(kl)) * 16) + (x & 7) * 2; b_sw[j] = 0;
#endif
  }
  const int frag_col = lane >> 5;

  // Fragment registers: wave tiles of 8 or more MFMAs per step keep one set and refill it
  // on the fly (the A fragment of row i is dead after its last column, the B fragment of
  // column j after the last row); smaller ones keep two sets.
#ifndef POLY_FRAG_ROLL
#define POLY_FRAG_ROLL (POLY_TM * POLY_TN >= 8)
#endif
  poly_in8 fa[POLY_FRAG_ROLL ? 1 : 2][POLY_TM], fb[POLY_FRAG_ROLL ? 1 : 2][POLY_TN];
  auto read_tr = [&](const unsigned char *p, int pitch) {
    // two transposing reads: k .. k+3 and k+4 .. k+7 of this lane's half of the 16-deep step
    union { poly_s16x4 h[2]; poly_in8 v; } u;
    u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((poly_lds_s16x4 *)p);
    u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((poly_lds_s16x4 *)(p + 4 * pitch));
    return u.v;
  };
  auto read_a = [&](int stage, int ks, int buf, int i) {
    const unsigned char *t = lds_raw + stage * POLY_STAGE_BYTES;
#if POLY_A_KC
    fa[buf][i] = *(const poly_in8 *)(t + a_fr[i] + (((ks * 2 + frag_col) ^ a_sw[i]) * 16));
#else
    fa[buf][i] = read_tr(t + a_fr[i] + ks * 16 * (POLY_BM * 2), POLY_BM * 2);
#endif
  };
  auto read_b = [&](int stage, int ks, int buf, int j) {
    const unsigned char *t = lds_raw + stage * POLY_STAGE_BYTES + POLY_A_BYTES;
#if POLY_B_KC
    fb[buf][j] = *(const poly_in8 *)(t + b_fr[j] + (((ks * 2 + frag_col) ^ b_sw[j]) * 16));
#else
    fb[buf][j] = read_tr(t + b_fr[j] + ks * 16 * (POLY_BN * 2), POLY_BN * 2);
#endif
  };
  auto read_frags = [&](int stage, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < POLY_TM; i++) read_a(stage, ks, buf, i);
#pragma unroll
    for (int j = 0; j < POLY_TN; j++) read_b(stage, ks, buf, j);
  };

  // One K tile: KS steps of MT MFMAs = KS * MT slots; each slot issues one MFMA, the
  // fragment refills that became possible, and its share of the LDS loads of a later tile.
  constexpr int KS = POLY_BK / 16, MT = POLY_TM * POLY_TN;
  auto k_tile = [&](int stage, auto &&slot_work) {
    read_frags(stage, 0, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      constexpr int R = POLY_FRAG_ROLL;
      if (!R && ks + 1 < KS) read_frags(stage, ks + 1, (ks + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < POLY_TM; i++)
#pragma unroll
        for (int j = 0; j < POLY_TN; j++) {
          const int buf = R ? 0 : (ks & 1);
          acc[i][j] = POLY_MFMA(fa[buf][i], fb[buf][j], acc[i][j]);
          if (R && ks + 1 < KS) {
            if (j == POLY_TN - 1) read_a(stage, ks + 1, 0, i);
            if (i == POLY_TM - 1) read_b(stage, ks + 1, 0, j);
          }
          slot_work(ks * MT + i * POLY_TN + j);
          __builtin_amdgcn_sched_barrier(0);
        }
    }
  };

  // ── the K loop ──────────────────────────────────────────────────────────────
  // Tile t lives in stage t % STAGES.  Iteration kt: wait until this wave's loads of tile
  // kt have landed (everything but the loads of the STAGES - 2 tiles issued after it),
  // barrier (every wave's part of tile kt is in LDS, and every wave is done reading tile
  // kt - 1), then multiply tile kt while issuing the loads of tile kt + STAGES - 1 into the
  // stage tile kt - 1 has just left.
#pragma unroll
  for (int t = 0; t < S - 1; t++)
    if (t < POLY_KT) issue_tile(t, t);
#ifdef POLY_EP_WIN_BYTES
  // unit u of the window's loads (issued during iteration KT - S + 1)
  auto issue_win_unit = [&](int u) {
    const int i = u * POLY_NW + wave;
    if (WIN_NI % POLY_NW != 0 && i >= WIN_NI) return;        // (wave-uniform)
    const int b = i * 1024 + lane * 16;
    const unsigned char *src = POLY_EP_WIN_SRC(b < POLY_EP_WIN_BYTES ? b : 0);
    const unsigned lds = lds_base + (unsigned)(WIN_STAGE * POLY_STAGE_BYTES) + (unsigned)i * 1024u;
    poly_lds_load_flat(lds, src);
  };
#endif
  // `vm`: loads issued after those of tile kt that may still be in flight; `ld`: this
  // iteration issues tile kt + S - 1; `win`: this iteration issues the window
  auto iteration = [&](int kt, int stage, int vm, bool ld, bool win) {
    poly_wait_vm(vm);
    __builtin_amdgcn_s_barrier();
    constexpr int SLOTS = KS * MT;
    k_tile(stage, [&](int slot) {
      if (ld) {
#pragma unroll
        for (int u = 0; u < POLY_IPW; u++)
          if (u * SLOTS / POLY_IPW == slot) issue_unit(u, kt + S - 1, (stage + S - 1) % S);
      }
#ifdef POLY_EP_WIN_BYTES
      if (win) {
#pragma unroll
        for (int u = 0; u < WIN_IPW; u++)
          if (u * SLOTS / WIN_IPW == slot) issue_win_unit(u);
      }
#endif
    });
  };
  // steady state: whole turns of the stage ring with every load present
  constexpr int STEADY = POLY_KT >= S ? ((POLY_KT - (S - 1)) / S) * S : 0;
  for (int kt = 0; kt < STEADY; kt += S) {
#pragma unroll
    for (int s = 0; s < S; s++) iteration(kt + s, s, (S - 2) * POLY_IPW, true, false);
  }
#pragma unroll
  for (int kt = STEADY; kt < POLY_KT; kt++) {
    // tiles after kt whose loads have been issued by now: min(S - 2, KT - 1 - kt); the
    // window's loads are younger than every tile's
    const int rest = POLY_KT - 1 - kt, later = rest < S - 2 ? rest : S - 2;
    const bool win_issued = WIN_IPW > 0 && kt > POLY_KT - S + 1;
    iteration(kt, kt % S, later * POLY_IPW + (win_issued ? WIN_IPW : 0), kt + S - 1 < POLY_KT, WIN_IPW > 0 && kt == POLY_KT - S + 1);
  }
  if (WIN_IPW > 0) poly_wait_vm(0);      // the window has landed (the barrier below publishes it)

  // ── epilogue ────────────────────────────────────────────────────────────────
  // Accumulator layout of the 32x32 MFMA: register r of lane l holds row
  // 8*(r/4) + 4*(l/32) + r%4, column l%32.  Each 32x32 tile goes through a per-wave LDS
  // staging area and comes back with 8 consecutive columns of one row per lane.
#if !POLY_EP_CONTIG && POLY_N % 8 != 0
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
  __syncthreads();   // every wave is done reading the operand tiles
  float *const stage = (float *)(lds_raw + OUT_OFF) + wave * (32 * POLY_STAGE_LD);
#pragma unroll
  for (int i = 0; i < POLY_TM; i++)
#pragma unroll
    for (int j = 0; j < POLY_TN; j++) {
#pragma unroll
      for (int r = 0; r < 16; r++)
        stage[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * POLY_STAGE_LD + (lane & 31)] = acc[i][j][r];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#ifdef POLY_EP_BLOCKMAX_LO
      typedef unsigned short poly_u16x8 __attribute__((ext_vector_type(8)));
      poly_u16x8 tile_mag = (poly_u16x8)(0);      // largest magnitudes as 16-bit patterns (ordered like the values, a NaN above all)
      const bool tile_counts = n0 + wn + j * 32 >= (POLY_EP_BLOCKMAX_LO) && n0 + wn + j * 32 < (POLY_EP_BLOCKMAX_HI);   // (wave-uniform)
#endif
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int row = (lane >> 2) + 16 * h, c0 = (lane & 3) * 8;
        const poly_f32x4 lo = *(const poly_f32x4 *)(stage + row * POLY_STAGE_LD + c0);
        const poly_f32x4 hi = *(const poly_f32x4 *)(stage + row * POLY_STAGE_LD + c0 + 4);
        const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const int m = m0 + wm + i * 32 + row, n = n0 + wn + j * 32 + c0;
#if POLY_EP_CONTIG
        if (m < POLY_M && n < POLY_N) {
          typedef POLY_EP_TYPE poly_out8 __attribute__((ext_vector_type(8)));
          typedef poly_out8 poly_out8_u __attribute__((aligned(sizeof(POLY_EP_TYPE))));
          poly_out8 o;
#if defined(POLY_EP_WIN_BYTES) && defined(POLY_EP_VALUE_WIN)
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
            const int ne = (POLY_N % 8 == 0 || n + e < POLY_N) ? n + e : n;
            o[e] = POLY_EP_VALUE(v[e], m, ne, z);
          }
#ifdef POLY_EP_BLOCKMAX_LO
          if (tile_counts) tile_mag = __builtin_elementwise_max(tile_mag, __builtin_bit_cast(poly_u16x8, o) & (poly_u16x8)(0x7fff));
#endif
          if (POLY_N % 8 == 0 || n + 7 < POLY_N) {
#ifdef POLY_EP_NT
            __builtin_nontemporal_store(o, (poly_out8_u *)POLY_EP_PTR(m, n, z));
#else
            *(poly_out8_u *)POLY_EP_PTR(m, n, z) = o;
#endif
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
#ifdef POLY_EP_BLOCKMAX_LO
      if (tile_counts) {
        unsigned int mag = tile_mag[0];
#pragma unroll
        for (int e = 1; e < 8; e++) mag = mag < tile_mag[e] ? (unsigned int)tile_mag[e] : mag;
        // the largest of each row of 16 lanes (register exchanges only), then one LDS atomic per row
#ifndef POLY_HOST_ADDRESS_CHECK
#define POLY_ROW_MAX_STEP(CTRL) { const unsigned int o_ = (unsigned int)__builtin_amdgcn_update_dpp(0, (int)mag, CTRL, 0xf, 0xf, true); mag = mag < o_ ? o_ : mag; }
        POLY_ROW_MAX_STEP(0xB1) POLY_ROW_MAX_STEP(0x4E) POLY_ROW_MAX_STEP(0x141) POLY_ROW_MAX_STEP(0x140)
#undef POLY_ROW_MAX_STEP
#endif
        // (as the bits of the float of that magnitude)
        const unsigned int tile_bits = __builtin_bit_cast(unsigned int, (float)__builtin_bit_cast(POLY_EP_TYPE, (unsigned short)mag));
        if ((lane & 15) == 0) atomicMax(&poly_blk[((wm + i * 32) / 64) * BLK_N + (wn + j * 32) / 64], tile_bits);
      }
#endif
    }
#ifdef POLY_EP_BLOCKMAX_LO
  if (n0 < (POLY_EP_BLOCKMAX_HI) && n0 + POLY_BN > (POLY_EP_BLOCKMAX_LO)) __syncthreads();      // (the same for the whole workgroup)
  if (threadIdx.x < BLK_COUNT) {
    const int bm0 = m0 + ((int)threadIdx.x / BLK_N) * 64, bn0 = n0 + ((int)threadIdx.x % BLK_N) * 64;
    if (bm0 < POLY_M && bn0 >= (POLY_EP_BLOCKMAX_LO) && bn0 < (POLY_EP_BLOCKMAX_HI)) (POLY_EP_BLOCKMAX_PTR)[POLY_EP_BLOCKMAX_IDX(bm0, bn0)] = poly_blk[threadIdx.x];
  }
#endif
#endif
}
