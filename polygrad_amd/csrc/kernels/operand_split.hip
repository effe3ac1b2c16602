// operand_split.hip -- writes one computed matmul operand as bf16 planes the 16-bit MFMA
// template can stream: OUT[z][row][part][k], rows of POLY_SP_PARTS * POLY_SP_KP elements,
// k-contiguous, zero for k >= POLY_SP_K.
//
// An fp32 value x is cut into three bf16 pieces hi + mid + lo (each the bf16 rounding of
// what the previous ones left over; the two residuals are exact in fp32 and the last
// rounding is below 2^-25 |x|).  A bf16 x bf16 product is exact in fp32, so
//     sum_k x[k] * b[k]  =  sum over the 3 K_p-long planes of  piece[k'] * b[k' mod K_p]
// on the bf16 MFMA with fp32 accumulation carries the same information as the fp32
// product at about a third of the bf16 rate (the fp32 MFMA runs at a sixteenth).  An
// operand that is a 16-bit value cast to fp32 is written as the single plane it is.
//
// Configuration (prepended by templates.cc):
//   POLY_SP_ROWS / POLY_SP_K / POLY_SP_Z   operand extents (rows = M or N)
//   POLY_SP_KP                             K rounded up to the K tile of the matmul
//   POLY_SP_PARTS                          3 (fp32 value) or 1 (already a bf16 value)
//   POLY_SP_WALK_K                         1: the source is contiguous along k, 0: along rows
//   POLY_SP_NRAW, POLY_SP_LOAD(row, k, z, raw), POLY_SP_MATH(row, k, z, raw)
//                                          the operand as the computed-operand matmul has it
//   POLY_SP_OUT                            the kernel argument that receives the planes
//   POLY_SIGNATURE
//
// One workgroup of 256 threads handles a 64 (rows) x 64 (k) tile: values are computed
// with lanes along whichever axis the source is contiguous in, pass through LDS, and
// leave with lanes along k.
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
  __shared__ float tile[64][65];
  constexpr int TILES_K = POLY_SP_KP / 64;
  const int tk = blockIdx.x % TILES_K, tr = blockIdx.x / TILES_K, z = blockIdx.y;
  const int row0 = tr * 64, k0 = tk * 64;
  // 16 elements per thread
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
  __bf16 *const out = (POLY_SP_OUT) + (size_t)z * POLY_SP_ROWS * (POLY_SP_PARTS * POLY_SP_KP);
#pragma unroll 4
  for (int i = 0; i < 16; i++) {
    const int c = threadIdx.x + i * 256;
    const int lr = c / 64, lk = c % 64;
    const int row = row0 + lr;
    if (row >= POLY_SP_ROWS) continue;
    const float x = tile[lr][lk];
    __bf16 *const dst = out + (size_t)row * (POLY_SP_PARTS * POLY_SP_KP) + k0 + lk;
    const __bf16 hi = (__bf16)x;
    dst[0] = hi;
    if (POLY_SP_PARTS == 3) {
      // (an infinite or NaN x is all in hi: no inf - inf in the residuals)
      const float r1 = __builtin_isfinite((float)hi) ? x - (float)hi : 0.0f;
      const __bf16 mid = (__bf16)r1;
      const float r2 = r1 - (float)mid;
      dst[POLY_SP_KP] = mid;
      dst[2 * POLY_SP_KP] = (__bf16)r2;
    }
  }
}
