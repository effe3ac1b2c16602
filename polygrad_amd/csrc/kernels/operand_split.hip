// operand_split.hip -- writes one computed matmul operand as bf16 planes the 16-bit MFMA
// template can stream: OUT[z][row][part][k], rows of POLY_SP_PARTS * POLY_SP_KP elements,
// k-contiguous, zero for k >= POLY_SP_K.
//
// An fp32 value x is cut into three bf16 pieces hi + mid + lo (each the bf16 rounding of
// what the previous ones left over; the two residuals are exact in fp32 and the last
// rounding is below 2^-25 |x|), or into the first two of them (what is left is below
// 2^-17 |x|) for a product whose result is stored as a 16-bit float.  A bf16 x bf16 product is exact in fp32, so
//     sum_k x[k] * b[k]  =  sum over the 3 K_p-long planes of  piece[k'] * b[k' mod K_p]
// on the bf16 MFMA with fp32 accumulation carries the same information as the fp32
// product at about a third of the bf16 rate (the fp32 MFMA runs at a sixteenth).  An
// operand that is a 16-bit value cast to fp32 is written as the single plane it is.
//
// Configuration (prepended by templates.cc):
//   POLY_SP_ROWS / POLY_SP_K / POLY_SP_Z   operand extents (rows = M or N)
//   POLY_SP_KP                             K rounded up to the K tile of the matmul
//   POLY_SP_PARTS                          3 or 2 (fp32 value) or 1 (already a bf16 value)
//   POLY_SP_WALK_K                         1: the source is contiguous along k, 0: along rows
//   POLY_SP_NRAW, POLY_SP_LOAD(row, k, z, raw), POLY_SP_MATH(row, k, z, raw)
//                                          the operand as the computed-operand matmul has it
//   POLY_SP_OUT                            the kernel argument that receives the planes
//   POLY_SIGNATURE
//
// One workgroup of 256 threads handles a 64 (rows) x 64 (k) tile, 16 values per thread: two
// groups of 8 neighbours along k when the source is contiguous in k and K a multiple of 8;
// otherwise with lanes along the source's contiguous axis and through LDS, to leave with
// lanes along k.
#ifdef POLY_TEMPLATE_STANDALONE
#include <hip/hip_runtime.h>
#define POLY_SP_ROWS 4096
#define POLY_SP_K 1000
#define POLY_SP_KP 1024
#define POLY_SP_Z 1
#define POLY_SP_PARTS 3
#define POLY_SP_WALK_K 0
#define POLY_SP_NRAW 1
#define POLY_SP_LOAD(row, k, z, raw) raw[0] = __builtin_bit_cast(unsigned int, data1[(k) * POLY_SP_ROWS + (row)])
#define POLY_SP_MATH(row, k, z, raw) __builtin_bit_cast(float, raw[0])
#define POLY_SP_OUT poly_planes
#define POLY_SIGNATURE float *data0, const float *__restrict__ data1, __bf16 *poly_planes
#endif

extern "C" __global__ void __launch_bounds__(256) poly_k(POLY_SIGNATURE) {
  constexpr int TILES_K = POLY_SP_KP / 64;
  const int tk = blockIdx.x % TILES_K, tr = blockIdx.x / TILES_K, z = blockIdx.y;
  const int row0 = tr * 64, k0 = tk * 64;
  __bf16 *const out = (POLY_SP_OUT) + (size_t)z * POLY_SP_ROWS * (POLY_SP_PARTS * POLY_SP_KP);
  typedef __bf16 sp_out8 __attribute__((ext_vector_type(8)));
  // 8 consecutive k of one row leave as one 16-byte store per plane (rows of the planes
  // start on multiples of 64 elements from a 256-byte aligned base)
  auto write_planes = [&](int row, int lk, const float (&x)[8]) {
    __bf16 *const dst = out + (size_t)row * (POLY_SP_PARTS * POLY_SP_KP) + k0 + lk;
    sp_out8 hi, mid, lo;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      hi[e] = (__bf16)x[e];
      if (POLY_SP_PARTS >= 2) {
        // (an infinite or NaN x is all in hi: no inf - inf in the residuals)
        const float r1 = __builtin_isfinite((float)hi[e]) ? x[e] - (float)hi[e] : 0.0f;
        mid[e] = (__bf16)r1;
        lo[e] = (__bf16)(r1 - (float)mid[e]);
      }
    }
    *(sp_out8 *)dst = hi;
    if (POLY_SP_PARTS >= 2) *(sp_out8 *)(dst + POLY_SP_KP) = mid;
    if (POLY_SP_PARTS == 3) *(sp_out8 *)(dst + 2 * POLY_SP_KP) = lo;
  };
#if POLY_SP_WALK_K && POLY_SP_K % 8 == 0
  // along k, rows a multiple of 8 long: a thread takes 8 neighbours, so that what the operand's expression loads for
  // them sits side by side and can be fetched together, and they are a row's piece as the
  // planes store it: no exchange needed
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int g = threadIdx.x + i * 256;
    const int lr = g / 8, lk = (g % 8) * 8;
    const int row = row0 + lr;
    if (row >= POLY_SP_ROWS) continue;
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int k = k0 + lk + e;
      x[e] = 0.0f;
      if (k < POLY_SP_K) {
        unsigned int raw[POLY_SP_NRAW];
        POLY_SP_LOAD(row, k, z, raw);
        x[e] = POLY_SP_MATH(row, k, z, raw);
      }
    }
    write_planes(row, lk, x);
  }
#else
  // along the rows, or along rows of k of any length: lanes along that axis (64 neighbours
  // per load), through LDS, to leave with lanes along k
  __shared__ float tile[64][65];
#pragma unroll 4
  for (int i = 0; i < 16; i++) {
    const int c = threadIdx.x + i * 256;
    const int lr = POLY_SP_WALK_K ? c / 64 : c % 64, lk = POLY_SP_WALK_K ? c % 64 : c / 64;
    const int row = row0 + lr, k = k0 + lk;
    float v = 0.0f;
    if (row < POLY_SP_ROWS && k < POLY_SP_K) {
      unsigned int raw[POLY_SP_NRAW];
      POLY_SP_LOAD(row, k, z, raw);
      v = POLY_SP_MATH(row, k, z, raw);
    }
    tile[lr][lk] = v;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int g = threadIdx.x + i * 256;
    const int lr = g / 8, lk = (g % 8) * 8;
    const int row = row0 + lr;
    if (row >= POLY_SP_ROWS) continue;
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] = tile[lr][lk + e];
    write_planes(row, lk, x);
  }
#endif
}
