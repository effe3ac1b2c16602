// Fused attention for gfx950: the kernel group
//     S = Q K^T  ->  pointwise chain (scale, mask, ...)  ->  row max  ->  row sum of
//     exp-terms  ->  normalise  ->  O = P V
// that a scheduler emits as six or more kernels, executed as one launch that never
// writes the [Z, M, N] score tensor to memory.  Only the STRUCTURE is fixed here; all
// arithmetic on scores (epilogue of the first matmul, the pointwise chain, the term
// that is summed, the normalisation, the epilogue of the second matmul) is generated
// from the kernels' own graphs and arrives through the POLY_FA_* hooks, rounding steps
// included, so every probability is computed by the same expression as in the unfused
// kernels.
//
// Two forms.  The exact form (below, POLY_FA_ONLINE 0) reproduces every rounding step of
// the unfused kernels; the online form (POLY_FA_ONLINE 1, further down) is the usual
// single-pass streaming softmax.
//
// Exact form: two passes over the keys.  Pass 1 computes each row's maximum and the sum of its terms
// (running maximum with rescaling; the hooks guarantee term(x, m) = exp2((x - m) * c),
// which makes the rescaling factor term(m_old, m_new)).  Pass 2 recomputes the scores
// (bit-identical: same MFMA sequence), turns them into probabilities with the final
// maximum and sum, and accumulates P V.
//
// Orientation: a wave owns 32 queries.  Scores are computed transposed,
// S^T[key][query] = K Q^T, so a lane holds ONE query (lane % 32) and 16 keys per 32x32
// tile in its accumulator registers: row statistics are in-register reductions plus one
// exchange between lane l and l ^ 32, and the probabilities are already laid out as the
// A operand of the second MFMA (8 keys per lane per 16-key step, in the key order
// 8*(i/4) + 4*(lane/32) + i%4 that the V fragment reads mirror).
//
// Configuration (defined by the host before this text):
//   POLY_TIN, POLY_MFMA(a, b, c)       16-bit input type and its 32x32x16 MFMA
//   POLY_FA_M, POLY_FA_N, POLY_FA_Z    queries, keys, batch*heads; M % 128 == 0, N % 64 == 0
//   POLY_Q_PTR, POLY_K_PTR, POLY_V_PTR operand pointers (names from POLY_SIGNATURE)
//   poly_q_off(z, m), poly_k_off(z, n), poly_v_off(z, n)
//                                      element offset of the 64 contiguous head features
//   POLY_FA_SCORE(acc, m, n, z)        -> POLY_TIN  score as the last pointwise kernel stores it
//   POLY_FA_MAXV(x, m, n, z)           -> float     what the max reduction compares
//   POLY_FA_TERM(x, mx, m, n, z)       -> float     what the sum reduction adds
//   POLY_FA_P(x, mx, sum, m, n, z)     -> POLY_TIN  the probability as stored
//   POLY_FA_OUT(acc, m, d, z)          stores one output element
//   POLY_FA_SKIP_DEAD_BLOCKS           1 when p = cast(term(x, mx) / sum): then a key block whose
//                                      terms are all exactly 0 has probabilities exactly 0
//   POLY_SIGNATURE
//   POLY_FA_MASK_PTR(m, n, z), POLY_FA_SCORE_MASK(acc, mk, m, n, z), POLY_FA_SCORE_NOMASK(acc, m, n, z)
//                                      (optional, online form, bf16) the score is
//                                      cast(f(acc) + mask) with f non-decreasing: address of
//                                      the mask entry (consecutive for consecutive n), the
//                                      score given the entry, and f(acc) as a float
//   POLY_FA_ONLINE                     1: single pass (needs p = cast(term / sum),
//                                      term(x, mx) = exp2((x - mx) * POLY_FA_C) and the
//                                      maximum taken over the scores themselves)
//   POLY_FA_QSCALE                     (optional, with POLY_FA_MASK_PTR) a power of two that
//                                      the kernel multiplies Q by when it stages it; the
//                                      score hooks are then generated without it
//   POLY_FA_MASK_TABLE                 (optional, with POLY_FA_MASK_PTR, when the mask does
//                                      not depend on z) pointer to the words that the
//                                      classifying kernel below writes: the mask is then
//                                      looked at once for all z instead of by every wave
//   POLY_FA_KMAX_TABLE                 (optional, with POLY_FA_MASK_TABLE) pointer to one word per
//                                      (z, block of 64 keys), [Z][N/64]: the bits of a float
//                                      that no feature of any key of the block exceeds in
//                                      magnitude (left there by the kernel that wrote the
//                                      keys).  A tile whose mask entries are all one value
//                                      is then passed over before its products when even
//                                      the score of kmax * sum |q| is dead
//   POLY_FA_CLASSIFY                   compile the classifying kernel instead of the
//                                      attention kernel (same configuration block, the
//                                      same arguments)
//
// Online form: one pass.  Per 32-key tile a wave computes the scores x exactly as the
// pointwise chain stores them (POLY_FA_SCORE, roundings included), the new running
// maximum m of each query, t = exp2((x - m) * c) in fp32, rescales the running sum and
// the output accumulators by exp2((m_old - m) * c) when a maximum moved, and accumulates
// O^T += V^T cast(t)^T; the division by the sum happens once at the end.  Against the
// unfused kernels the 16-bit rounding of the probabilities moves from t / sum to t (the
// output differs from theirs by about one 16-bit rounding).  A key tile whose mask entries
// are all -inf is passed over before its scores, and one whose terms are all exact zeros
// against the running maxima after them: a non-finite product or V under probabilities
// that are all zero does not propagate.
// The output is transposed relative to the exact form: a lane holds ONE query in both
// MFMAs, so maximum, sum and rescaling factor are per-lane scalars.
//
// Dead key blocks (every term of the block exactly zero for all 32 queries of a wave, as
// under a causal mask) are detected from the values themselves, never assumed: term is
// monotone in x, so term(block maximum, row maximum) == 0 bounds the whole block.  Pass 1
// then skips the exponentials of that block (they would add exact zeros) and pass 2 skips
// its scores and probabilities, multiplying V by exact zeros instead so that a non-finite
// V still propagates as it does in the unfused kernels.  Blocks with a NaN score are
// never treated as dead.
#ifdef POLY_TEMPLATE_STANDALONE
#include <hip/hip_runtime.h>
#define POLY_TIN __bf16
#define POLY_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)
#define POLY_FA_M 1024
#define POLY_FA_N 1024
#define POLY_FA_Z 96
#define POLY_Q_PTR data1
#define POLY_K_PTR data2
#define POLY_V_PTR data3
#ifdef POLY_STANDALONE_QKV   // q, k, v as column blocks of one [8192, 2304] buffer
__device__ __forceinline__ int poly_q_off(int z, int m) { return (z / 12) * 2359296 + (z % 12) * 64 + m * 2304; }
__device__ __forceinline__ int poly_k_off(int z, int n) { return (z / 12) * 2359296 + (z % 12) * 64 + n * 2304 + 768; }
__device__ __forceinline__ int poly_v_off(int z, int n) { return (z / 12) * 2359296 + (z % 12) * 64 + n * 2304 + 1536; }
#else
__device__ __forceinline__ int poly_q_off(int z, int m) { return (z / 12) * 786432 + (z % 12) * 64 + m * 768; }
__device__ __forceinline__ int poly_k_off(int z, int n) { return (z / 12) * 786432 + (z % 12) * 64 + n * 768; }
__device__ __forceinline__ int poly_v_off(int z, int n) { return (z / 12) * 786432 + (z % 12) * 64 + n * 768; }
#endif
#ifdef POLY_STANDALONE_MASK_TABLE
#define POLY_SIGNATURE __bf16 *data0, const __bf16 *__restrict__ data1, const __bf16 *__restrict__ data2, const __bf16 *__restrict__ data3, const __bf16 *__restrict__ data4, unsigned int *poly_scratch
#define POLY_FA_MASK_TABLE poly_scratch
#else
#define POLY_SIGNATURE __bf16 *data0, const __bf16 *__restrict__ data1, const __bf16 *__restrict__ data2, const __bf16 *__restrict__ data3, const __bf16 *__restrict__ data4
#endif
#define POLY_FA_SCORE(acc, m, n, z) ((__bf16)((float)(__bf16)(acc) * 0.125f + (float)data4[(m) * 1024 + (n)]))
#define POLY_FA_MAXV(x, m, n, z) ((float)(x))
#define POLY_FA_TERM(x, mx, m, n, z) __builtin_amdgcn_exp2f(((float)(x) - (mx)) * 0x1.715476p+0f)
#define POLY_FA_P(x, mx, sum, m, n, z) ((__bf16)(__builtin_amdgcn_exp2f(((float)(x) - (mx)) * 0x1.715476p+0f) / (sum)))
#define POLY_FA_OUT(acc, m, d, z) data0[((z) / 12) * 786432 + ((z) % 12) * 65536 + (m) * 64 + (d)] = (__bf16)(acc)
#define POLY_FA_SKIP_DEAD_BLOCKS 1
#define POLY_FA_ONLINE 1
#define POLY_FA_C 0x1.715476p+0f
#define POLY_FA_MASK_PTR(m, n, z) (data4 + (m) * 1024 + (n))
#define POLY_FA_QSCALE 0.125f
#define POLY_FA_SCORE_MASK(acc, mk, m, n, z) ((__bf16)((float)(__bf16)(acc) + (float)(mk)))
#define POLY_FA_SCORE_NOMASK(acc, m, n, z) ((float)(__bf16)(acc))
#endif
#ifndef POLY_FA_ONLINE
#define POLY_FA_ONLINE 0
#endif

typedef POLY_TIN fa_in8 __attribute__((ext_vector_type(8)));
typedef float fa_acc16 __attribute__((ext_vector_type(16)));
typedef unsigned int fa_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int fa_u32x2 __attribute__((ext_vector_type(2)));
typedef fa_u32x4 fa_u32x4_u __attribute__((aligned(2)));
typedef fa_u32x2 fa_u32x2_u __attribute__((aligned(2)));

#ifndef POLY_FA_OCC
#define POLY_FA_OCC 3    // waves per SIMD the register budget is set for (a tuning candidate: no effect on the values)
#endif
#define FA_BM 128        // queries per workgroup: 4 waves x 32
#define FA_BN 64         // keys per step
#define FA_D 64          // head features
#define FA_THREADS 256
#define FA_NKB (POLY_FA_N / FA_BN)
#ifndef FA_LAG
#define FA_LAG 8.0f      // online form: how many powers of two a score may exceed the reference before it moves
#endif

// LDS tiles are [row][64] 16-bit values; the eight 16-byte columns of a row are
// XOR-swizzled by the row number so fragment reads and staging writes spread over banks.
__device__ __forceinline__ int fa_swz(int row) { return (row ^ (row >> 3)) & 7; }

__device__ __forceinline__ float fa_other_half(float v) {
  // value held by lane ^ 32: v_permlane32_swap exchanges lanes 32..63 of its first operand
  // with lanes 0..31 of its second (written as assembly: the compiler's builtin for it
  // returned the first exchange's result for every later one)
#ifdef POLY_HOST_ADDRESS_CHECK   // the kernel compiled for the host to check its indexing: lanes run one by one
  return v;
#else
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return (threadIdx.x & 32) ? a : b;
#endif
}

#ifdef POLY_FA_CLASSIFY
// The kernel that looks at a z-independent mask once for all z (see POLY_FA_MASK_TABLE
// below for the layout it writes).  One workgroup of 8 waves per block of 128 queries x
// 64 keys, one wave per 32 x 32 tile.
extern "C" __global__ void __launch_bounds__(512) poly_k(POLY_SIGNATURE) {
  __shared__ int dead_tiles;
  if (threadIdx.x == 0) dead_tiles = 0;
  __syncthreads();
  constexpr int NB = POLY_FA_N / 64;
  const int rb = blockIdx.x / NB, cb = blockIdx.x % NB;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int qt = 4 * rb + (wave >> 1), kt = 2 * cb + (wave & 1);
  fa_u32x4 look[2];
#pragma unroll
  for (int i = 0; i < 2; i++) look[i] = *(const fa_u32x4_u *)POLY_FA_MASK_PTR(32 * qt + 16 * i + (lane >> 2), 32 * kt + 8 * (lane & 3), 0);
  const unsigned s0 = (unsigned)__builtin_amdgcn_readfirstlane((int)((look[0][0] & 0xffffu) * 0x10001u));
  unsigned diff = 0;
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) diff |= look[i][j] ^ s0;
  const bool uniform = __builtin_amdgcn_ballot_w64(diff != 0) == 0;
  unsigned *const table = (unsigned *)(POLY_FA_MASK_TABLE);
  if (lane == 0) {
    table[qt * (POLY_FA_N / 32) + kt] = (s0 & 0xffffu) | (uniform ? 0x10000u : 0u);
    if (uniform && __builtin_bit_cast(float, s0 << 16) == -__builtin_inff()) atomicAdd(&dead_tiles, 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) table[(POLY_FA_M / 32) * (POLY_FA_N / 32) + rb * NB + cb] = dead_tiles == 8 ? 1u : 0u;
}
#else
// Three workgroups per CU (three waves per SIMD): the arithmetic on the scores is VALU work,
// and it is the other resident waves that hide its latencies.
extern "C" __global__ void __launch_bounds__(FA_THREADS) __attribute__((amdgpu_waves_per_eu(POLY_FA_OCC, POLY_FA_OCC))) poly_k(POLY_SIGNATURE) {
  __shared__ __attribute__((aligned(16))) POLY_TIN lds_k[2][FA_BN * FA_D];   // [key][feature]
  __shared__ __attribute__((aligned(16))) POLY_TIN lds_v[2][FA_D * FA_BN];   // [feature][key]
  __shared__ __attribute__((aligned(16))) POLY_TIN lds_q[FA_BM * FA_D];      // [query][feature]

  // Workgroup -> (z, block of queries).  Consecutive ids go to different XCDs (id % 8), each
  // with its own L2: an XCD keeps a fixed set of z, so the query blocks that share K and V
  // meet in one L2.  Under a causal mask late query blocks have more live key tiles than
  // early ones, so within an XCD the late blocks are handed out first.
  constexpr int MB = POLY_FA_M / FA_BM;
  int z, mb;
  if (POLY_FA_Z % 8 == 0) {
    constexpr int ZX = POLY_FA_Z / 8 > 0 ? POLY_FA_Z / 8 : 1;   // z per XCD
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
#ifdef POLY_FA_ORDER
    // (a table from the renderer: the same blocks, dealt so that the three workgroups that
    // share a CU carry about the same number of key blocks together)
    const int item = poly_fa_order[j];
    mb = item / ZX;
    z = xcd * ZX + item % ZX;
#else
    mb = MB - 1 - j / ZX;
    z = xcd * ZX + j % ZX;
#endif
  } else {
    mb = MB - 1 - (int)blockIdx.x / POLY_FA_Z;
    z = (int)blockIdx.x % POLY_FA_Z;
  }
  const int m0 = mb * FA_BM;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lq = lane & 31, half = lane >> 5;
  const int mq = m0 + wave * 32 + lq;   // the query this lane owns in the score tiles

  // Q block of the workgroup -> LDS once (128 queries x 8 chunks of 16 bytes, four per
  // thread); it is the B operand of S^T = K Q^T: a lane reads Q[mq][16 s + 8 half .. + 7]
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int c = threadIdx.x + i * FA_THREADS;
    const int q = c >> 3, col = c & 7;
    fa_u32x4 v = *(const fa_u32x4_u *)(POLY_Q_PTR + poly_q_off(z, m0 + q) + col * 8);
#ifdef POLY_FA_QSCALE
    // the power of two that the score chain would multiply every cast(acc) by, applied to Q
    {
      fa_in8 qv = __builtin_bit_cast(fa_in8, v);
#pragma unroll
      for (int e = 0; e < 8; e++) qv[e] = (POLY_TIN)((float)qv[e] * POLY_FA_QSCALE);
      v = __builtin_bit_cast(fa_u32x4, qv);
    }
#endif
    *(fa_u32x4 *)(lds_q + q * FA_D + ((col ^ fa_swz(q)) * 8)) = v;
  }
  const POLY_TIN *q_row = lds_q + (wave * 32 + lq) * FA_D;
  const int q_sw = fa_swz(wave * 32 + lq);

  // staging of K: 64 keys x 8 chunks of 16 bytes = 512 chunks, two per thread
  int k_key[2], k_col[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int c = threadIdx.x + i * FA_THREADS;
    k_key[i] = c >> 3;
    k_col[i] = c & 7;
  }
  auto load_k = [&](int kb, fa_u32x4 (&rk)[2]) {
#pragma unroll
    for (int i = 0; i < 2; i++)
      rk[i] = *(const fa_u32x4_u *)(POLY_K_PTR + poly_k_off(z, kb * FA_BN + k_key[i]) + k_col[i] * 8);
  };
  auto store_k = [&](int buf, const fa_u32x4 (&rk)[2]) {
#pragma unroll
    for (int i = 0; i < 2; i++)
      *(fa_u32x4 *)(lds_k[buf] + k_key[i] * FA_D + ((k_col[i] ^ fa_swz(k_key[i])) * 8)) = rk[i];
  };
  // staging of V: 4 keys x 8 features per thread (threads 0..127), transposed in
  // registers into 8 feature rows x 4 keys and written as 8-byte pieces
  const bool v_thread = threadIdx.x < 128;
  const int v_chunk = threadIdx.x & 7, v_kq = (threadIdx.x >> 3) & 15;   // features 8*chunk.., keys 4*kq..
  auto load_v = [&](int kb, fa_u32x4 (&rv)[4]) {
    if (v_thread) {
#pragma unroll
      for (int i = 0; i < 4; i++)
        rv[i] = *(const fa_u32x4_u *)(POLY_V_PTR + poly_v_off(z, kb * FA_BN + v_kq * 4 + i) + v_chunk * 8);
    }
  };
  auto store_v = [&](int buf, const fa_u32x4 (&rv)[4]) {
    if (v_thread) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        // dword j of load i holds features 2j (low half) and 2j+1 (high half) of key 4*kq+i
        const unsigned int a0 = rv[0][j], a1 = rv[1][j], a2 = rv[2][j], a3 = rv[3][j];
        fa_u32x2 lo, hi;
        lo[0] = (a0 & 0xffffu) | (a1 << 16);
        lo[1] = (a2 & 0xffffu) | (a3 << 16);
        hi[0] = (a0 >> 16) | (a1 & 0xffff0000u);
        hi[1] = (a2 >> 16) | (a3 & 0xffff0000u);
        const int r0 = v_chunk * 8 + 2 * j, r1 = r0 + 1;
        *(fa_u32x2 *)(lds_v[buf] + r0 * FA_BN + (((v_kq >> 1) ^ fa_swz(r0)) * 8) + (v_kq & 1) * 4) = lo;
        *(fa_u32x2 *)(lds_v[buf] + r1 * FA_BN + (((v_kq >> 1) ^ fa_swz(r1)) * 8) + (v_kq & 1) * 4) = hi;
      }
    }
  };

  // S^T tile of this wave: 32 keys (tile t of the staged block) x 32 queries
  auto scores = [&](int buf, int t, fa_acc16 &st) {
#pragma unroll
    for (int r = 0; r < 16; r++) st[r] = 0.0f;
    const int key = 32 * t + lq;
    const POLY_TIN *row = lds_k[buf] + key * FA_D;
    const int sw = fa_swz(key);
#pragma unroll
    for (int s = 0; s < FA_D / 16; s++) {
      const fa_in8 kf = *(const fa_in8 *)(row + (((2 * s + half) ^ sw) * 8));
      const fa_in8 qf = *(const fa_in8 *)(q_row + (((2 * s + half) ^ q_sw) * 8));
      st = POLY_MFMA(kf, qf, st);
    }
  };
  // key index of accumulator register r of tile t
  auto key_of = [&](int kb, int t, int r) { return kb * FA_BN + 32 * t + 8 * (r >> 2) + 4 * half + (r & 3); };

#if POLY_FA_ONLINE
  // ── online form: one pass over the keys ─────────────────────────────────────
  fa_acc16 o[2];
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
  float m_run = -__builtin_inff(), l_run = 0.0f;   // identical maximum on both lanes of a query; sum of this lane's keys
  {
    const float c = POLY_FA_C;
    fa_u32x4 rk[2], rv[4];
#ifdef POLY_FA_MASK_PTR
    // this lane's 16 keys of a tile: four runs of 4 consecutive keys, 8 bytes each (the
    // entries of one query are consecutive in memory)
    const POLY_TIN *const mask_row = POLY_FA_MASK_PTR(mq, 4 * half, z);
#endif
    float q_l1 = 0.0f;   // (with POLY_FA_KMAX_TABLE) sum of |q| over the features of this lane's query, as staged
    // One 32 x 32 tile: tile t of key block kb, staged in LDS buffer cur.  With a mask,
    // `uniform` says that all its 32 x 32 entries hold the one value `cmask`.
    auto tile = [&](int cur, int kb, int t, bool uniform, float cmask, float kmax) {
      // V^T fragment (A operand): feature row 32 dt + lq, the 8 keys of this lane's half
      // of the 16 keys 32t + 16u .., in the key order of the score registers
      auto v_frag = [&](int u, int dt) {
        const int col0 = 4 * t + 2 * u;
        const int d = 32 * dt + lq;
        const POLY_TIN *row = lds_v[cur] + d * FA_BN;
        const int sw = fa_swz(d);
        const fa_u32x2 lo = *(const fa_u32x2 *)(row + ((col0 ^ sw) * 8) + half * 4);
        const fa_u32x2 hi = *(const fa_u32x2 *)(row + (((col0 + 1) ^ sw) * 8) + half * 4);
        fa_u32x4 both;
        both[0] = lo[0]; both[1] = lo[1]; both[2] = hi[0]; both[3] = hi[1];
        return __builtin_bit_cast(fa_in8, both);
      };
      float x[16];
#ifdef POLY_FA_MASK_PTR
      // -inf everywhere: every score of the tile is -inf whatever the (finite) product,
      // every term an exact zero and no maximum moves; a query that has seen nothing but
      // such tiles keeps sum 0 and ends as 0 / 0 like in the unfused kernels.  (A
      // non-finite product goes unseen here: its key is masked out for every query of
      // the tile, and would have made the unfused kernels' rows NaN.)
      if (uniform && cmask == -__builtin_inff()) return;
#ifdef POLY_FA_KMAX_TABLE
      // One value is added everywhere and no key of the block has a feature larger than
      // kmax in magnitude: |product| <= kmax * sum |q| for every key (the factor covers
      // the roundings of both sums).  If even the score of that bound has a term of exactly
      // zero against the running maximum, for all 32 queries, the tile adds nothing and
      // moves no maximum, and its products are not computed.  (A non-finite kmax or query
      // makes the bound NaN or +inf, which is never dead.)
      if (uniform && cmask != 0.0f) {
        const int n0 = key_of(kb, t, 0);
        const float bound = POLY_FA_MAXV(POLY_FA_SCORE_MASK(q_l1 * kmax * 1.001f, (POLY_TIN)cmask, mq, n0, z), mq, n0, z);
        const bool early_dead = __builtin_amdgcn_exp2f((bound - m_run) * c) == 0.0f;
        if (__builtin_amdgcn_ballot_w64(!early_dead) == 0) return;
      }
#else
      (void)kmax;
#endif
      asm volatile("" ::: "memory");   // (keeps the fragment reads and MFMAs below the test)
      fa_acc16 st;
      scores(cur, t, st);
      if (uniform && cmask == 0.0f) {
        // nothing is added: the score is f(acc), already a 16-bit value
#pragma unroll
        for (int r = 0; r < 16; r++) x[r] = POLY_FA_SCORE_NOMASK(st[r], mq, key_of(kb, t, r), z);
      } else {
        if (uniform) {
          // One value c is added everywhere: the score of the largest product bounds this
          // lane's scores.  If even its term is an exact zero against the running maximum
          // for all 32 queries, the tile adds nothing and moves no maximum.  (A NaN product
          // goes unseen here, as above.)
          float amax = st[0];
#pragma unroll
          for (int r = 1; r < 16; r++) amax = __builtin_fmaxf(amax, st[r]);
          const int n0 = key_of(kb, t, 0);
          const float bound = POLY_FA_MAXV(POLY_FA_SCORE_MASK(amax, (POLY_TIN)cmask, mq, n0, z), mq, n0, z);
          const bool early_dead = __builtin_amdgcn_exp2f((bound - m_run) * c) == 0.0f;
          if (__builtin_amdgcn_ballot_w64(!early_dead) == 0) return;
        }
        // entries in the layout of the score registers
        fa_u32x2 mraw[4];
#pragma unroll
        for (int gq = 0; gq < 4; gq++) mraw[gq] = *(const fa_u32x2_u *)(mask_row + 32 * (2 * kb + t) + 8 * gq);
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int n = key_of(kb, t, r);
          const unsigned d = mraw[r >> 2][(r >> 1) & 1];
          const POLY_TIN mk = __builtin_bit_cast(POLY_TIN, (unsigned short)((r & 1) ? (d >> 16) : (d & 0xffffu)));
          x[r] = POLY_FA_MAXV(POLY_FA_SCORE_MASK(st[r], mk, mq, n, z), mq, n, z);
        }
      }
#else
      fa_acc16 st;
      scores(cur, t, st);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int n = key_of(kb, t, r);
        x[r] = POLY_FA_MAXV(POLY_FA_SCORE(st[r], mq, n, z), mq, n, z);
      }
#endif
      // largest score of this lane's keys; a NaN among them makes it NaN (v_maximum3_f32)
      float bm = x[0];
#pragma unroll
      for (int r = 1; r < 16; r++) bm = __builtin_elementwise_maximum(bm, x[r]);
      bm = __builtin_elementwise_maximum(bm, fa_other_half(bm));
      // Against the running maximum the largest term of this tile is exactly zero (the
      // exponential underflows, or the scores are -inf) for all 32 queries: the maxima
      // do not move and every term is an exact zero.  (A query with no finite score yet
      // has m_run = -inf and counts as live, and so does one with a NaN score: both make
      // the exponential NaN.)
      const float dist = (bm - m_run) * c;   // how far above the reference the tile reaches, in powers of two
      const bool lane_dead = __builtin_amdgcn_exp2f(dist) == 0.0f;
      if (__builtin_amdgcn_ballot_w64(!lane_dead) == 0) return;
      // m_run is the reference the terms are taken against.  It follows the largest score
      // lazily: only when some query's tile maximum lies more than 2^FA_LAG above it (or it
      // is still -inf, or a NaN is involved) do all queries of the wave move theirs, with
      // the usual rescaling of sum and accumulators; otherwise terms simply come out as
      // large as 2^FA_LAG, which fp32 sums and a 16-bit float hold as well as values below
      // one, and the final division takes out whatever reference was used.  After the
      // first tiles of a row this is rare, and the rescaling was a sixth of the tile's
      // vector instructions.
      const bool move = !(dist <= FA_LAG);
      if (__builtin_amdgcn_ballot_w64(move) != 0) {
        const float m_new = __builtin_fmaxf(m_run, bm);   // ignores a NaN: the terms carry it
        // a query whose keys were all -inf so far: subtract 0 instead (its terms come out 0,
        // not NaN; if the row stays empty the final 0 / 0 is the NaN the unfused kernels give)
        const float m_to = (m_new == -__builtin_inff()) ? 0.0f : m_new;
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_to) * c);
        l_run = l_run * alpha;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
          for (int dt = 0; dt < 2; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[dt][r] = o[dt][r] * alpha;
        }
      }
      // The exponent (x - m) c as one fused multiply-add, x c - (m c): the rounding of m c
      // puts 2^-24 |m c| into the exponent, which is nothing while the reference is of any
      // ordinary size (|m| <= 4096: 3.5e-4 at most, a tenth of the 16-bit rounding of the
      // term) and ruinous for scores of 1e9.  References beyond that (rare: one test per
      // tile, the same for the whole wave) take the difference first, as the unfused
      // kernels do.
      const float m_ref = (m_run == -__builtin_inff()) ? 0.0f : m_run;
      const float mc = m_ref * c;
      float sum = 0.0f;
      POLY_TIN p[16];
      if (__builtin_amdgcn_ballot_w64(!(__builtin_fabsf(m_ref) <= 4096.0f)) == 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float tt = __builtin_amdgcn_exp2f(__builtin_fmaf(x[r], c, -mc));
          sum = sum + tt;
          p[r] = (POLY_TIN)tt;
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float tt = __builtin_amdgcn_exp2f((x[r] - m_ref) * c);
          sum = sum + tt;
          p[r] = (POLY_TIN)tt;
        }
      }
      l_run = l_run + sum;
#pragma unroll
      for (int u = 0; u < 2; u++) {
        fa_in8 pf;
#pragma unroll
        for (int i = 0; i < 8; i++) pf[i] = p[8 * u + i];
#pragma unroll
        for (int dt = 0; dt < 2; dt++) o[dt] = POLY_MFMA(v_frag(u, dt), pf, o[dt]);
      }
    };
#ifdef POLY_FA_MASK_TABLE
    // The mask does not depend on z, and a kernel ahead of this one has looked at it once
    // for all z: POLY_FA_MASK_TABLE points at one word per 32 x 32 tile ([M/32][N/32]:
    // bit 16 set when all entries of the tile hold one value, that value in the low 16
    // bits), followed by one word per block of 128 queries x 64 keys ([M/128][N/64]:
    // non-zero when every entry of the block is -inf).  All of it is read through scalar
    // loads, and the key blocks that are -inf for the whole workgroup are neither loaded
    // nor waited for.
    const unsigned *const tile_words = (const unsigned *)(POLY_FA_MASK_TABLE) + (m0 / 32 + __builtin_amdgcn_readfirstlane(wave)) * (POLY_FA_N / 32);
    const unsigned *const block_words = (const unsigned *)(POLY_FA_MASK_TABLE) + (POLY_FA_M / 32) * (POLY_FA_N / 32) + mb * FA_NKB;
#if POLY_FA_N / 32 <= 64
    // up to 64 tiles along the keys: lane l fetches the word of tile l and of block l once,
    // and the loop below picks them out of the lanes (no load, no wait per tile)
    const unsigned my_tile_word = lane < POLY_FA_N / 32 ? tile_words[lane] : 0u;
    const unsigned my_block_word = lane < FA_NKB ? block_words[lane] : 1u;
    const unsigned long long live_blocks = __builtin_amdgcn_ballot_w64(my_block_word == 0u);
    auto tile_word = [&](int ti) { return (unsigned)__builtin_amdgcn_readlane((int)my_tile_word, ti); };
    auto next_block = [&](int kb) {
      const unsigned long long rest = kb < 64 ? (live_blocks >> kb) : 0ull;
      return rest ? kb + __builtin_ctzll(rest) : FA_NKB;
    };
#else
    auto tile_word = [&](int ti) { return tile_words[ti]; };
    auto next_block = [&](int kb) {
      while (kb < FA_NKB && block_words[kb] != 0) kb++;
      return kb;
    };
#endif
    int kb = next_block(0), cur = 0;
    if (kb < FA_NKB) {
      load_k(kb, rk);
      load_v(kb, rv);
      store_k(0, rk);
      store_v(0, rv);
    }
    __syncthreads();
#if defined(POLY_FA_KMAX_TABLE) && POLY_FA_N / 32 <= 64
    // lane l fetches the bound of key block l once (the bits of a float; whatever the
    // keys' product has not written reads as NaN, which bounds nothing)
    const unsigned my_kmax_bits = lane < FA_NKB ? (POLY_FA_KMAX_TABLE)[z * FA_NKB + lane] : 0xffffffffu;
#pragma unroll
    for (int ch = 0; ch < 8; ch++) {
      const fa_in8 qf = *(const fa_in8 *)(q_row + ch * 8);
#pragma unroll
      for (int e = 0; e < 8; e++) q_l1 += __builtin_fabsf((float)qf[e]);
    }
    // When every tile that is left has one non-zero mask value for all four waves, the
    // workgroup may be done before the last key block: each wave then tests the tiles left
    // against its queries all at once (lane l: tile l, with the largest sum |q| and the
    // smallest running maximum of the wave's queries), the waves tell each other through
    // LDS in front of the block's barrier, and when all four say so the loop ends there --
    // no load, store or barrier for the blocks behind.  Which blocks are left is the same
    // for the four waves (the mask words of all four rows of tiles are looked at), so all
    // of them take part in the same exchanges.
    __shared__ int fa_rest_dead[2][4];
    unsigned long long live_tiles, hard_tiles;
    {
      const unsigned *const wg_words = (const unsigned *)(POLY_FA_MASK_TABLE) + (m0 / 32) * (POLY_FA_N / 32);
      bool one_value = lane < POLY_FA_N / 32;
#pragma unroll
      for (int w = 0; w < 4; w++) {
        const unsigned u = lane < POLY_FA_N / 32 ? wg_words[w * (POLY_FA_N / 32) + lane] : 0u;
        one_value = one_value && (u >> 16) != 0 && (u & 0x7fffu) != 0;
      }
      live_tiles = __builtin_amdgcn_ballot_w64(lane < POLY_FA_N / 32 && ((live_blocks >> (lane >> 1)) & 1ull) != 0);
      hard_tiles = live_tiles & ~__builtin_amdgcn_ballot_w64(one_value);
    }
    const unsigned my_tile_kmax_bits = (unsigned)__builtin_amdgcn_ds_bpermute((lane >> 1) << 2, (int)my_kmax_bits);   // of the block of tile `lane`
    unsigned q1max_bits = __builtin_bit_cast(unsigned, q_l1);      // (sums of magnitudes: ordered like their bits, a NaN above all)
#pragma unroll
    for (int sh = 1; sh < 64; sh <<= 1) {
      const unsigned o = (unsigned)__builtin_amdgcn_ds_bpermute((lane ^ sh) << 2, (int)q1max_bits);
      q1max_bits = q1max_bits < o ? o : q1max_bits;
    }
    int turn = 0;
#endif
    while (kb < FA_NKB) {
      const int nb = next_block(kb + 1);
      if (nb < FA_NKB) { load_k(nb, rk); load_v(nb, rv); }
#if defined(POLY_FA_KMAX_TABLE) && POLY_FA_N / 32 <= 64
      const float kmax = __builtin_bit_cast(float, __builtin_amdgcn_readlane((int)my_kmax_bits, kb));
#else
      const float kmax = __builtin_inff();
#endif
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const unsigned w = tile_word(2 * kb + t);
        tile(cur, kb, t, (w >> 16) != 0, __builtin_bit_cast(float, w << 16), kmax);
      }
#if defined(POLY_FA_KMAX_TABLE) && POLY_FA_N / 32 <= 64
      const unsigned long long rest = 2 * (kb + 1) < 64 ? (live_tiles & (~0ull << (2 * (kb + 1)))) : 0ull;
      const bool exchange = rest != 0 && (hard_tiles & rest) == 0;      // (the same in all four waves)
      if (exchange) {
        float m_min = m_run;
#pragma unroll
        for (int sh = 1; sh < 64; sh <<= 1) m_min = __builtin_fminf(m_min, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ sh) << 2, __builtin_bit_cast(int, m_min))));
        const float ub = __builtin_bit_cast(float, q1max_bits) * __builtin_bit_cast(float, my_tile_kmax_bits) * 1.001f;
        const POLY_TIN mk = __builtin_bit_cast(POLY_TIN, (unsigned short)(my_tile_word & 0xffffu));
        const int n_of = 32 * (lane < POLY_FA_N / 32 ? lane : 0);
        const float bound = POLY_FA_MAXV(POLY_FA_SCORE_MASK(ub, mk, mq, n_of, z), mq, n_of, z);
        const bool lane_dead = __builtin_amdgcn_exp2f((bound - m_min) * c) == 0.0f;
        const bool mine = ((rest >> lane) & 1ull) != 0;
        const bool rest_dead = __builtin_amdgcn_ballot_w64(mine && !lane_dead) == 0;
        if (lane == 0) fa_rest_dead[turn][wave] = rest_dead ? 1 : 0;
      }
#endif
      if (nb < FA_NKB) { store_k(cur ^ 1, rk); store_v(cur ^ 1, rv); }
      __syncthreads();
#if defined(POLY_FA_KMAX_TABLE) && POLY_FA_N / 32 <= 64
      if (exchange) {
        const int all = fa_rest_dead[turn][0] & fa_rest_dead[turn][1] & fa_rest_dead[turn][2] & fa_rest_dead[turn][3];
        if (all) break;
      }
      turn ^= 1;
#endif
      kb = nb;
      cur ^= 1;
    }
#else
    load_k(0, rk);
    load_v(0, rv);
    store_k(0, rk);
    store_v(0, rv);
    __syncthreads();
#ifdef POLY_FA_MASK_PTR
    // Is the mask one value over a 32 x 32 tile?  Any lane can look at any entries for that,
    // so the tile is read the cheap way: 16 bytes per lane, four lanes along a query's 64
    // bytes, 16 queries per load (16 cache lines per instruction; in the layout of the
    // score registers, 8 bytes per lane with 32 queries per load, the same tile takes four
    // times as many line accesses, and those were what the memory pipeline spent its time
    // on).  The entries in score layout are fetched only for a tile that is not uniform.
    const POLY_TIN *const look_row0 = POLY_FA_MASK_PTR(m0 + wave * 32 + (lane >> 2), 8 * (lane & 3), z);
    const POLY_TIN *const look_row1 = POLY_FA_MASK_PTR(m0 + wave * 32 + 16 + (lane >> 2), 8 * (lane & 3), z);
    auto load_look = [&](int tl, fa_u32x4 (&lk)[2]) {
      lk[0] = *(const fa_u32x4_u *)(look_row0 + 32 * tl);
      lk[1] = *(const fa_u32x4_u *)(look_row1 + 32 * tl);
    };
    fa_u32x4 look[2];
    load_look(0, look);
#endif
    for (int kb = 0; kb < FA_NKB; kb++) {
      const int cur = kb & 1;
      if (kb + 1 < FA_NKB) { load_k(kb + 1, rk); load_v(kb + 1, rv); }
#ifdef POLY_FA_MASK_PTR
#pragma unroll
      for (int t = 0; t < 2; t++) {
        // the entries of the tile after this one are requested now, a tile ahead of their use
        fa_u32x4 look_next[2];
        load_look((2 * kb + t + 1 < 2 * FA_NKB) ? 2 * kb + t + 1 : 2 * kb + t, look_next);
        // Do all 32 x 32 entries hold one value?  (compared as bit patterns)
        const unsigned s0 = (unsigned)__builtin_amdgcn_readfirstlane((int)((look[0][0] & 0xffffu) * 0x10001u));
        unsigned diff = 0;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 4; j++) diff |= look[i][j] ^ s0;
        const bool uniform = __builtin_amdgcn_ballot_w64(diff != 0) == 0;
        tile(cur, kb, t, uniform, __builtin_bit_cast(float, s0 << 16), __builtin_inff());
        look[0] = look_next[0];
        look[1] = look_next[1];
      }
#else
      tile(cur, kb, 0, false, 0.0f, __builtin_inff());
      tile(cur, kb, 1, false, 0.0f, __builtin_inff());
#endif
      if (kb + 1 < FA_NKB) { store_k(cur ^ 1, rk); store_v(cur ^ 1, rv); }
      __syncthreads();
    }
#endif
  }
  // the two lanes of a query each summed half of the keys (a + b == b + a bit for bit)
  const float l_tot = l_run + fa_other_half(l_run);
  // O^T tile: register r of lane l holds feature 8*(r/4) + 4*(l/32) + r%4 of query l%32
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++)
      POLY_FA_OUT(o[dt][r] / l_tot, mq, 32 * dt + 8 * (r >> 2) + 4 * half + (r & 3), z);
#else
  // ── pass 1: row maximum and sum of terms, one 32-key tile at a time ─────────
  float row_max = -__builtin_inff(), row_sum = 0.0f;
  unsigned long long dead = 0;   // wave-uniform: 32-key tiles whose terms are all exactly zero
  {
    fa_u32x4 rk[2];
    load_k(0, rk);
    store_k(0, rk);
    __syncthreads();
    for (int kb = 0; kb < FA_NKB; kb++) {
      const int cur = kb & 1;
      if (kb + 1 < FA_NKB) load_k(kb + 1, rk);
#pragma unroll
      for (int t = 0; t < 2; t++) {
        fa_acc16 st;
        scores(cur, t, st);
        POLY_TIN x[16];
        float bm = -__builtin_inff(), nan_probe = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int n = key_of(kb, t, r);
          x[r] = POLY_FA_SCORE(st[r], mq, n, z);
          const float v = POLY_FA_MAXV(x[r], mq, n, z);
          bm = __builtin_fmaxf(bm, v);   // like (bm < v) ? v : bm, a NaN v is ignored
          nan_probe = nan_probe + v;      // NaN if any value is (or +inf meets -inf: then not skipped)
        }
        const float new_max = (row_max < bm) ? bm : row_max;
        // nothing but -inf so far for this lane's half of the keys: its sum stays 0 and its
        // maximum -inf (terms against a maximum of -inf would be NaN; if the other half of
        // the row has a finite score these keys get probability 0, otherwise the row is
        // NaN as in the unfused kernels, which the merge below produces)
        const bool empty = (new_max == -__builtin_inff()) && (nan_probe == nan_probe);
        // upper bound of this lane's terms in this tile
        const float bound = POLY_FA_TERM((POLY_TIN)bm, new_max, mq, 0, z);
        const bool lane_dead = empty || ((bound == 0.0f) && (nan_probe == nan_probe));
        if (__builtin_amdgcn_ballot_w64(!lane_dead) != 0) {
          float acc = row_sum * POLY_FA_TERM((POLY_TIN)row_max, new_max, mq, 0, z);
#pragma unroll
          for (int r = 0; r < 16; r++) acc = acc + POLY_FA_TERM(x[r], new_max, mq, key_of(kb, t, r), z);
          if (!empty) {
            row_sum = acc;
            row_max = new_max;
          }
        } else {
          // every term is an exact zero and the maximum did not move: nothing to add
          if (2 * kb + t < 64) dead |= 1ull << (2 * kb + t);
        }
      }
      if (kb + 1 < FA_NKB) store_k(cur ^ 1, rk);
      __syncthreads();
    }
    // the two lanes of a query (l, l ^ 32) each saw half of the keys
    const float o_max = fa_other_half(row_max), o_sum = fa_other_half(row_sum);
    const float f_max = (row_max < o_max) ? o_max : row_max;
    const float mine = row_sum * POLY_FA_TERM((POLY_TIN)row_max, f_max, mq, 0, z);
    const float theirs = o_sum * POLY_FA_TERM((POLY_TIN)o_max, f_max, mq, 0, z);
    // same operand order on both lanes, so both hold the identical sum
    row_sum = half == 0 ? mine + theirs : theirs + mine;
    row_max = f_max;
  }

  // ── pass 2: probabilities and P V ───────────────────────────────────────────
  fa_acc16 o[2];
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
  {
    // zero / sum is an exact zero only for a finite, non-zero sum
    const bool sums_ok = __builtin_amdgcn_ballot_w64(!(row_sum > 0.0f && row_sum < __builtin_inff())) == 0;
    fa_u32x4 rk[2], rv[4];
    load_k(0, rk);
    load_v(0, rv);
    store_k(0, rk);
    store_v(0, rv);
    __syncthreads();
    for (int kb = 0; kb < FA_NKB; kb++) {
      const int cur = kb & 1;
      if (kb + 1 < FA_NKB) { load_k(kb + 1, rk); load_v(kb + 1, rv); }
      // V fragment (B operand) for the 16 keys 32t + 16u .. of feature tile dt
      auto v_frag = [&](int t, int u, int dt) {
        const int col0 = 4 * t + 2 * u;   // 16-byte column of keys 32t+16u .. +7 in a V^T row
        const int d = 32 * dt + lq;
        const POLY_TIN *row = lds_v[cur] + d * FA_BN;
        const int sw = fa_swz(d);
        const fa_u32x2 lo = *(const fa_u32x2 *)(row + ((col0 ^ sw) * 8) + half * 4);
        const fa_u32x2 hi = *(const fa_u32x2 *)(row + (((col0 + 1) ^ sw) * 8) + half * 4);
        fa_u32x4 both;
        both[0] = lo[0]; both[1] = lo[1]; both[2] = hi[0]; both[3] = hi[1];
        return __builtin_bit_cast(fa_in8, both);
      };
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int tile = 2 * kb + t;
        const bool skip = POLY_FA_SKIP_DEAD_BLOCKS && sums_ok && tile < 64 && ((dead >> tile) & 1ull);
        if (skip) {
          // probabilities are exact zeros; 0 * V keeps a non-finite V visible
          fa_in8 zf;
#pragma unroll
          for (int i = 0; i < 8; i++) zf[i] = (POLY_TIN)0.0f;
#pragma unroll
          for (int u = 0; u < 2; u++)
#pragma unroll
            for (int dt = 0; dt < 2; dt++) o[dt] = POLY_MFMA(zf, v_frag(t, u, dt), o[dt]);
        } else {
          fa_acc16 st;
          scores(cur, t, st);
          POLY_TIN p[16];
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int n = key_of(kb, t, r);
            const POLY_TIN x = POLY_FA_SCORE(st[r], mq, n, z);
            p[r] = POLY_FA_P(x, row_max, row_sum, mq, n, z);
          }
#pragma unroll
          for (int u = 0; u < 2; u++) {
            fa_in8 pf;
#pragma unroll
            for (int i = 0; i < 8; i++) pf[i] = p[8 * u + i];
#pragma unroll
            for (int dt = 0; dt < 2; dt++) o[dt] = POLY_MFMA(pf, v_frag(t, u, dt), o[dt]);
          }
        }
      }
      if (kb + 1 < FA_NKB) { store_k(cur ^ 1, rk); store_v(cur ^ 1, rv); }
      __syncthreads();
    }
  }

  // Output tile: register r of lane l holds query row 8*(r/4) + 4*(l/32) + r%4, feature l%32.
#pragma unroll
  for (int dt = 0; dt < 2; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int m = m0 + wave * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
      POLY_FA_OUT(o[dt][r], m, 32 * dt + lq, z);
    }
#endif
}
#endif
