// Shared pieces of the int4 dequantising matmul kernels: the argument block,
// the pre-tiled weight layout, nibble -> f16 conversion and the matching
// permutation of the activations.
#ifndef IREE_AMD_UK_I4_H_
#define IREE_AMD_UK_I4_H_

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace uk {
namespace i4 {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;               // K-slices per workgroup
constexpr int kThreads = kWaves * 64;

struct I4Args {
  const uint16_t* x;      // [M][K] f16
  const uint8_t* w;       // u4, tiled or row-major
  const uint16_t* scale;  // [N][G] f16
  const void* zp;         // [N][G] f16 or packed u4
  uint16_t* out;          // [M][N] f16
  int M, N, K, G;
  int log2_gs;            // group size = 1 << log2_gs
  int zp_u4;
  int tiled;
  int n_tiles;            // ceil(N / 32)
  int m_base;             // first activation row of this pass
  int stage_rows;         // rows the LDS staging area of a wave holds (8 or 16), 16-row form
  // weight addressing of the fast kernel: byte offset of the 16 bytes that
  // lane (nl, kc) reads for column c of tile nt in 128-k span s is
  //   nt * K * 16 + s * span_stride + c * col_stride + kc * 16
  uint32_t span_stride, col_stride;
  uint32_t w_bytes;       // size of the weight buffer
  // A K longer than one workgroup takes (512 KB elements): workgroup row
  // blockIdx.y multiplies the y-th slice of so many elements and, with more
  // than one row, stores its f32 sums at partial[(y * M + m) * N + n] for a
  // second kernel to add in row order (nullptr: one row, f16 results to out).
  float* partial;
};

// Position, in the tiled layout, of the byte that holds elements (n, k) and
// (n, k+1), k even. A tile is 32 columns by 128 k (2 KiB): 64 bytes per column,
// in which the 16 dwords of the row-major span are transposed as a 4 x 4
// matrix, so that 16-byte chunk kc holds, as dword q, k = q*32 + kc*8 .. +8.
__host__ __device__ inline size_t tiled_byte_index(int64_t n, int64_t k, int64_t K) {
  const int64_t s = k >> 7, r = k & 127, q = r >> 5, kc = (r >> 3) & 3, j = r & 7;
  return (size_t)((((n >> 5) * (K >> 7) + s) * 32 + (n & 31)) * 64 + kc * 16 + q * 4 + (j >> 1));
}

// 8 nibbles of one dword -> 8 small f16 integers (nibble - zero point), in the
// k order [0,4,1,5,2,6,3,7] of the dword's nibbles (pairs (i, i+4) fall out of
// one AND/OR); the activation operand is permuted the same way. `lo` is
// 1024 + zp and `hi` 64 + zp as packed f16 pairs: 0x6400 | n is 1024 + n and
// 0x6400 | (n << 4) is 1024 + 16 n, so (1024 + n) - lo and
// (1024 + 16 n) / 16 - hi are both n - zp, every step exact for integer zp.
// (w & mask) | 0x6400'6400 in ONE instruction. The compiler will not form
// v_and_or_b32 from the C expression because two 32-bit literals do not fit
// one instruction; with the mask in a vector register it does.
__device__ __forceinline__ uint32_t and_or_magic(uint32_t w, uint32_t mask) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(w), "v"(mask), "s"(0x64006400u));
  return r;
}

__device__ __forceinline__ half8 dequant_dword(uint32_t w, half2v lo, half2v hi) {
  union { uint32_t u; half2v h; } a, b, c, d;
  const uint32_t w8 = w >> 8;
  a.u = and_or_magic(w, 0x000F000Fu);    // nibbles 0, 4
  b.u = and_or_magic(w, 0x00F000F0u);    // nibbles 1, 5 (x16)
  c.u = and_or_magic(w8, 0x000F000Fu);   // nibbles 2, 6
  d.u = and_or_magic(w8, 0x00F000F0u);   // nibbles 3, 7 (x16)
  const half2v sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  const half2v r0 = a.h - lo, r1 = b.h * sixteenth - hi, r2 = c.h - lo, r3 = d.h * sixteenth - hi;
  return half8{r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
}

// The cheaper form, used where the register file has room for the group sums
// of the activations: the nibbles go to the matrix cores as f16 SUBNORMALS.
// w & 0x000F000F is the pair (n0, n4) * 2^-24 and w & 0x00F000F0 the pair
// (n1, n5) * 16 * 2^-24 (v_mfma_f32_16x16x32_f16 takes subnormal inputs at full
// precision, and a subnormal times an f16 is exact in f32), so 8 weights cost
// one shift and four ANDs. The activations that meet the second kind are
// divided by 16 beforehand (permute_x_for_subnormals), and the zero point
// leaves the inner loop altogether: sum_k x (n - zp) = sum_k x n - zp sum_k x,
// with the group sums of x taken once per workgroup.
__device__ __forceinline__ half8 nibbles_as_subnormals(uint32_t w) {
  union { uint32_t u[4]; half8 h; } r;
  const uint32_t w8 = w >> 8;
  r.u[0] = w & 0x000F000Fu;     // nibbles 0, 4
  r.u[1] = w & 0x00F000F0u;     // nibbles 1, 5 (x16)
  r.u[2] = w8 & 0x000F000Fu;    // nibbles 2, 6
  r.u[3] = w8 & 0x00F000F0u;    // nibbles 3, 7 (x16)
  return r.h;
}
// What the products of that operand have to be multiplied by.
constexpr float kSubnormalUnit = 5.9604644775390625e-8f;      // 2^-24
constexpr float kSubnormalRescale = 16777216.0f;              // 2^24

// The two offsets for a packed uint4 zero point zp (0..15), as f16 pairs:
// 1024 + zp = 0x6400 | zp and 64 + zp = 0x5400 | (zp << 4) (ulp 1/16 at 64).
__device__ __forceinline__ uint32_t offset_lo_bits(uint32_t zp) { return 0x64006400u | zp | (zp << 16); }
__device__ __forceinline__ uint32_t offset_hi_bits(uint32_t zp) { return 0x54005400u | (zp << 4) | (zp << 20); }

// x[m][k .. k+8) (8 consecutive halves, 16 bytes) -> the same 8 halves in the
// order [0,4,1,5,2,6,3,7].
__device__ __forceinline__ half8 permute_x(u32x4 v) {
  union { uint32_t u[4]; half8 h; } r;
  // v.x = (h0,h1) v.y = (h2,h3) v.z = (h4,h5) v.w = (h6,h7)
  r.u[0] = __builtin_amdgcn_perm(v.z, v.x, 0x05040100);  // (h0, h4)
  r.u[1] = __builtin_amdgcn_perm(v.z, v.x, 0x07060302);  // (h1, h5)
  r.u[2] = __builtin_amdgcn_perm(v.w, v.y, 0x05040100);  // (h2, h6)
  r.u[3] = __builtin_amdgcn_perm(v.w, v.y, 0x07060302);  // (h3, h7)
  return r.h;
}

// The same, with the halves that meet nibbles held 16-fold (positions 2, 3, 6,
// 7 of the permuted order) divided by 16: exact down to 2^-10, below that the
// quotient is rounded to the subnormal grid (an absolute error of at most
// 2^-25 per activation).
__device__ __forceinline__ half8 permute_x_for_subnormals(u32x4 v) {
  union { half8 h; half2v p[4]; } r;
  r.h = permute_x(v);
  const half2v sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  r.p[1] = r.p[1] * sixteenth;
  r.p[3] = r.p[3] * sixteenth;
  return r.h;
}
// The constant operand whose product with such activations is their plain sum.
__device__ __forceinline__ half8 ones_for_subnormal_sums() {
  return half8{(_Float16)1.f, (_Float16)1.f, (_Float16)16.f, (_Float16)16.f,
               (_Float16)1.f, (_Float16)1.f, (_Float16)16.f, (_Float16)16.f};
}

// NB bytes (1 .. 16 naturally aligned, 32 aligned to 16) into NB/4 (at least 1) dwords.
template <int NB>
__device__ __forceinline__ void load_bits(const void* p, uint32_t* dst) {
  if constexpr (NB == 1) dst[0] = *(const uint8_t*)p;
  else if constexpr (NB == 2) dst[0] = *(const uint16_t*)p;
  else if constexpr (NB == 4) dst[0] = *(const uint32_t*)p;
  else if constexpr (NB == 8) { const u32x2 v = *(const u32x2*)p; dst[0] = v.x; dst[1] = v.y; }
  else if constexpr (NB == 16) { const u32x4 v = *(const u32x4*)p; dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w; }
  else { static_assert(NB == 32, "unsupported width"); load_bits<16>(p, dst); load_bits<16>((const uint8_t*)p + 16, dst + 4); }
}

}  // namespace i4

// Rows [m_base, m_base + m_eff), m_eff <= 16, through the per-wave-column kernel
// (uk_quant_gemv.hip); IREE_AMD_UK_STATUS_NOT_FOUND for shapes it does not take.
int launch_dequant_gemv_i4(const i4::I4Args& p, int m_base, int m_eff, hipStream_t s);

}  // namespace uk

#endif  // IREE_AMD_UK_I4_H_
