// Affine 8-bit row quantiser / dequantiser and the cache-slot write for gfx950 (HBM-bound byte work).
//
// Reference behaviour: keys_values/kvcache/quantize/pytorch.py:100-139,312-355 (quantise),
// :143-154,411-478 (dequantise); keys_values/kvcache/attn_weights.py:305-316,679-681 and
// keys_values/kvcache/buffers.py:498-519 (slot write).
//
// A row of D bf16 values is spread over D/8 adjacent lanes, 8 values (one 16-byte load) per lane,
// so a wavefront reads 1 KiB of contiguous input per load instruction and writes 512 contiguous
// bytes of codes. Row min and max are reduced with DPP moves inside the 16-lane row (no LDS).
#include "kvx_common.h"

namespace kvx {
namespace {

constexpr int NTHREADS = 256;
constexpr int ROWS_PER_THREAD = 4;  // independent rows in flight per lane

// Reductions over the LPR (8, 16 or 32) adjacent lanes holding one row; every lane gets the result.
template <int LPR>
__device__ __forceinline__ float row_max(float v) {
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true)));   // quad_perm [1,0,3,2]
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true)));   // quad_perm [2,3,0,1]
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true)));  // row_half_mirror
  if constexpr (LPR >= 16)
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true)));  // row_mirror
  if constexpr (LPR == 32) v = fmaxf(v, __shfl_xor(v, 16, 64));  // the other DPP row of the group
  return v;
}
template <int LPR>
__device__ __forceinline__ float row_min(float v) {
  v = fminf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true)));
  v = fminf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true)));
  v = fminf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true)));
  if constexpr (LPR >= 16)
    v = fminf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true)));
  if constexpr (LPR == 32) v = fminf(v, __shfl_xor(v, 16, 64));
  return v;
}

// Does one of the 8 values hold a NaN? The reference takes a row's extremes with torch.aminmax
// (keys_values/kvcache/quantize/pytorch.py:90), which returns NaN for a row that holds one: such a row
// gets a NaN scale and dequantises to NaN throughout (fminf / fmaxf would drop the NaN).
__device__ __forceinline__ bool has_nan8(const float (&x)[8]) {
  return __builtin_isunordered(x[0], x[1]) | __builtin_isunordered(x[2], x[3]) | __builtin_isunordered(x[4], x[5]) |
         __builtin_isunordered(x[6], x[7]);
}

// True in all LPR lanes of a row if one of them says `bad`. The wavefront's ballot is a scalar: rows
// with a NaN are rare, and the test costs a scalar compare when there is none.
template <int LPR>
__device__ __forceinline__ bool row_any(bool bad) {
  const unsigned long long m = __ballot(bad);
  if (m == 0) return false;
  const int first = (int)(__lane_id() & ~(unsigned)(LPR - 1));
  return ((m >> first) & ((1ull << LPR) - 1ull)) != 0;
}

// Codes of 4 values packed into a dword, byte e = clamp(rint(x[e] * inv) + zf, 0, 255). The sum is an
// integer-valued float, so the conversion's rounding does not matter; v_cvt_pk_u8_f32 saturates to
// [0, 255] (a NaN gives 0) and places the byte, which is the clamp, the cast and the packing in one.
__device__ __forceinline__ uint32_t codes4_u8(float x0, float x1, float x2, float x3, float inv, float zf) {
  uint32_t w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(x0 * inv) + zf, 0, 0);
  w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(x1 * inv) + zf, 1, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(x2 * inv) + zf, 2, w);
  return __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(x3 * inv) + zf, 3, w);
}
// The same with codes clamped to [0, 15] (4-bit store).
__device__ __forceinline__ uint32_t codes4_u4(float x0, float x1, float x2, float x3, float inv, float zf) {
  uint32_t w = __builtin_amdgcn_cvt_pk_u8_f32(fminf(__builtin_rintf(x0 * inv) + zf, 15.0f), 0, 0);
  w = __builtin_amdgcn_cvt_pk_u8_f32(fminf(__builtin_rintf(x1 * inv) + zf, 15.0f), 1, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(fminf(__builtin_rintf(x2 * inv) + zf, 15.0f), 2, w);
  return __builtin_amdgcn_cvt_pk_u8_f32(fminf(__builtin_rintf(x3 * inv) + zf, 15.0f), 3, w);
}

template <int LPR, bool F16>
__device__ __forceinline__ void row_extremes(u32x4_t raw, float (&x)[8], float& mn, float& mx) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[2 * e] = elem_lo<F16>(raw[e]);
    x[2 * e + 1] = elem_hi<F16>(raw[e]);
  }
  mn = x[0];
  mx = x[0];
#pragma unroll
  for (int e = 1; e < 8; ++e) {
    mn = fminf(mn, x[e]);
    mx = fmaxf(mx, x[e]);
  }
  mn = row_min<LPR>(mn);
  mx = row_max<LPR>(mx);
  if (row_any<LPR>(has_nan8(x))) mn = mx = __builtin_nanf("");
}

// The ROWS_PER_THREAD rows a lane works on at once share the per-row arithmetic (three IEEE divisions):
// all lanes of a row hold its extremes, so lane c of a quad works out the scale and zero point of row
// c only, and the others fetch 1 / scale and the zero point from it with a quad broadcast. Returns the
// codes of row i in c[i] (bytes), and in (scale, zp) the state of row (lane & 3).
template <int LPR, int BITS, bool F16>
__device__ __forceinline__ void quantize_rows_in_flight(const u32x4_t (&raw)[ROWS_PER_THREAD], u32x2_t (&c)[ROWS_PER_THREAD], float& scale,
                                                        int32_t& zp) {
  static_assert(ROWS_PER_THREAD == 4, "one row per lane of a quad");
  float x[ROWS_PER_THREAD][8], mn[ROWS_PER_THREAD], mx[ROWS_PER_THREAD];
#pragma unroll
  for (int i = 0; i < ROWS_PER_THREAD; ++i) row_extremes<LPR, F16>(raw[i], x[i], mn[i], mx[i]);
  const int mine = (int)(__lane_id() & 3u);
  const float my_mn = mine == 0 ? mn[0] : mine == 1 ? mn[1] : mine == 2 ? mn[2] : mn[3];
  const float my_mx = mine == 0 ? mx[0] : mine == 1 ? mx[1] : mine == 2 ? mx[2] : mx[3];
  quant_params(my_mn, my_mx, scale, zp, BITS == 8 ? 255.0f : 15.0f);
  const int inv_bits = __builtin_bit_cast(int, 1.0f / scale);
  const int zf_bits = __builtin_bit_cast(int, (float)zp);
  float inv[ROWS_PER_THREAD], zf[ROWS_PER_THREAD];
  inv[0] = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(inv_bits, 0x00, 0xf, 0xf, true));  // quad_perm [0,0,0,0]
  inv[1] = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(inv_bits, 0x55, 0xf, 0xf, true));  // quad_perm [1,1,1,1]
  inv[2] = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(inv_bits, 0xAA, 0xf, 0xf, true));  // quad_perm [2,2,2,2]
  inv[3] = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(inv_bits, 0xFF, 0xf, 0xf, true));  // quad_perm [3,3,3,3]
  zf[0] = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(zf_bits, 0x00, 0xf, 0xf, true));
  zf[1] = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(zf_bits, 0x55, 0xf, 0xf, true));
  zf[2] = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(zf_bits, 0xAA, 0xf, 0xf, true));
  zf[3] = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(zf_bits, 0xFF, 0xf, 0xf, true));
#pragma unroll
  for (int i = 0; i < ROWS_PER_THREAD; ++i) {
    if constexpr (BITS == 8) {
      c[i][0] = codes4_u8(x[i][0], x[i][1], x[i][2], x[i][3], inv[i], zf[i]);
      c[i][1] = codes4_u8(x[i][4], x[i][5], x[i][6], x[i][7], inv[i], zf[i]);
    } else {
      c[i][0] = codes4_u4(x[i][0], x[i][1], x[i][2], x[i][3], inv[i], zf[i]);
      c[i][1] = codes4_u4(x[i][4], x[i][5], x[i][6], x[i][7], inv[i], zf[i]);
    }
  }
}

// Quantise the 8 values of this lane's share of a row; every lane of the row returns the same
// scale / zero point.
template <int LPR, bool F16>
__device__ __forceinline__ u32x2_t quantize8(u32x4_t raw, float& scale, int32_t& zp) {
  float x[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[2 * e] = elem_lo<F16>(raw[e]);
    x[2 * e + 1] = elem_hi<F16>(raw[e]);
  }
  float mn = x[0], mx = x[0];
#pragma unroll
  for (int e = 1; e < 8; ++e) {
    mn = fminf(mn, x[e]);
    mx = fmaxf(mx, x[e]);
  }
  mn = row_min<LPR>(mn);
  mx = row_max<LPR>(mx);
  if (row_any<LPR>(has_nan8(x))) mn = mx = __builtin_nanf("");  // aminmax propagates NaN, fminf / fmaxf drop it
  quant_params(mn, mx, scale, zp);
  const float inv = 1.0f / scale;
  const float zf = (float)zp;
  u32x2_t out;
  out[0] = quant_code(x[0], inv, zf) | (quant_code(x[1], inv, zf) << 8) | (quant_code(x[2], inv, zf) << 16) |
           (quant_code(x[3], inv, zf) << 24);
  out[1] = quant_code(x[4], inv, zf) | (quant_code(x[5], inv, zf) << 8) | (quant_code(x[6], inv, zf) << 16) |
           (quant_code(x[7], inv, zf) << 24);
  return out;
}

template <int D, bool F16>
__global__ __launch_bounds__(NTHREADS) void quantize_rows_kernel(const uint16_t* __restrict__ x, int64_t x_row_stride,
                                                                 int64_t rows, uint8_t* __restrict__ codes,
                                                                 float* __restrict__ scale, int32_t* __restrict__ zp) {
  constexpr int LPR = D / 8;
  constexpr int RPB = NTHREADS / LPR;  // rows per block per step
  const int col = threadIdx.x % LPR;
  const int64_t row0 = (int64_t)blockIdx.x * (RPB * ROWS_PER_THREAD) + threadIdx.x / LPR;
  u32x4_t raw[ROWS_PER_THREAD];
#pragma unroll
  for (int i = 0; i < ROWS_PER_THREAD; ++i) {
    const int64_t r = row0 + (int64_t)i * RPB;
    raw[i] = r < rows ? __builtin_nontemporal_load((const u32x4_t*)(x + r * x_row_stride + col * 8)) : u32x4_t{0, 0, 0, 0};
  }
  u32x2_t c[ROWS_PER_THREAD];
  float s;
  int32_t z;
  quantize_rows_in_flight<LPR, 8, F16>(raw, c, s, z);  // executed by all lanes: the DPP exchanges need them
#pragma unroll
  for (int i = 0; i < ROWS_PER_THREAD; ++i) {
    const int64_t r = row0 + (int64_t)i * RPB;
    if (r < rows) *(u32x2_t*)(codes + r * D + col * 8) = c[i];
  }
  // lane `col` of a row's first quad holds the state of row `col` of the four
  const int64_t r_mine = row0 + (int64_t)col * RPB;
  if (col < ROWS_PER_THREAD && r_mine < rows) {
    scale[r_mine] = s;
    zp[r_mine] = z;
  }
}

template <int D, bool F16>
__global__ __launch_bounds__(NTHREADS) void dequantize_rows_kernel(const uint8_t* __restrict__ codes,
                                                                   const float* __restrict__ scale,
                                                                   const int32_t* __restrict__ zp, int64_t rows,
                                                                   uint16_t* __restrict__ out, int64_t out_row_stride) {
  constexpr int LPR = D / 8;
  constexpr int RPB = NTHREADS / LPR;
  const int col = threadIdx.x % LPR;
  const int64_t row0 = (int64_t)blockIdx.x * (RPB * ROWS_PER_THREAD) + threadIdx.x / LPR;
  u32x2_t c[ROWS_PER_THREAD];
  float s[ROWS_PER_THREAD];
  int32_t z[ROWS_PER_THREAD];
#pragma unroll
  for (int i = 0; i < ROWS_PER_THREAD; ++i) {
    const int64_t r = row0 + (int64_t)i * RPB;
    const bool ok = r < rows;
    c[i] = ok ? *(const u32x2_t*)(codes + r * D + col * 8) : u32x2_t{0, 0};
    s[i] = ok ? scale[r] : 0.0f;
    z[i] = ok ? zp[r] : 0;
  }
#pragma unroll
  for (int i = 0; i < ROWS_PER_THREAD; ++i) {
    const int64_t r = row0 + (int64_t)i * RPB;
    if (r >= rows) continue;
    *(u32x4_t*)(out + r * out_row_stride + col * 8) = dequant_words<F16>(c[i][0], c[i][1], z[i], s[i]);
  }
}

// ---- 4-bit rows -------------------------------------------------------------------------------

// Codes of the lane's 8 values as bytes (0..15), same layout as quantize8.
template <int LPR, bool F16>
__device__ __forceinline__ u32x2_t quantize4(u32x4_t raw, float& scale, int32_t& zp) {
  float x[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[2 * e] = elem_lo<F16>(raw[e]);
    x[2 * e + 1] = elem_hi<F16>(raw[e]);
  }
  float mn = x[0], mx = x[0];
#pragma unroll
  for (int e = 1; e < 8; ++e) {
    mn = fminf(mn, x[e]);
    mx = fmaxf(mx, x[e]);
  }
  mn = row_min<LPR>(mn);
  mx = row_max<LPR>(mx);
  if (row_any<LPR>(has_nan8(x))) mn = mx = __builtin_nanf("");  // aminmax propagates NaN, fminf / fmaxf drop it
  quant_params(mn, mx, scale, zp, 15.0f);
  const float inv = 1.0f / scale;
  const float zf = (float)zp;
  u32x2_t out;
  out[0] = quant_code(x[0], inv, zf, 15.0f) | (quant_code(x[1], inv, zf, 15.0f) << 8) | (quant_code(x[2], inv, zf, 15.0f) << 16) |
           (quant_code(x[3], inv, zf, 15.0f) << 24);
  out[1] = quant_code(x[4], inv, zf, 15.0f) | (quant_code(x[5], inv, zf, 15.0f) << 8) | (quant_code(x[6], inv, zf, 15.0f) << 16) |
           (quant_code(x[7], inv, zf, 15.0f) << 24);
  return out;
}

// Element d shares its byte with element d + D/2 (high nibble = first half of the row): the lanes of
// the first half fetch their partner's codes from the lane LPR/2 away and store 8 packed bytes.
template <int D, bool F16>
__global__ __launch_bounds__(NTHREADS) void quantize_rows4_kernel(const uint16_t* __restrict__ x, int64_t x_row_stride, int64_t rows,
                                                                  uint8_t* __restrict__ codes, float* __restrict__ scale,
                                                                  int32_t* __restrict__ zp) {
  constexpr int LPR = D / 8;
  constexpr int RPB = NTHREADS / LPR;
  const int col = threadIdx.x % LPR;
  const int64_t row0 = (int64_t)blockIdx.x * (RPB * ROWS_PER_THREAD) + threadIdx.x / LPR;
  u32x4_t raw[ROWS_PER_THREAD];
#pragma unroll
  for (int i = 0; i < ROWS_PER_THREAD; ++i) {
    const int64_t r = row0 + (int64_t)i * RPB;
    raw[i] = r < rows ? __builtin_nontemporal_load((const u32x4_t*)(x + r * x_row_stride + col * 8)) : u32x4_t{0, 0, 0, 0};
  }
  u32x2_t c[ROWS_PER_THREAD];
  float s;
  int32_t z;
  quantize_rows_in_flight<LPR, 4, F16>(raw, c, s, z);  // executed by all lanes: the reductions and the exchanges need them
#pragma unroll
  for (int i = 0; i < ROWS_PER_THREAD; ++i) {
    const int64_t r = row0 + (int64_t)i * RPB;
    const uint32_t p0 = __shfl_xor(c[i][0], LPR / 2, 64), p1 = __shfl_xor(c[i][1], LPR / 2, 64);
    if (r < rows && col < LPR / 2) *(u32x2_t*)(codes + r * (D / 2) + col * 8) = u32x2_t{(c[i][0] << 4) | p0, (c[i][1] << 4) | p1};
  }
  const int64_t r_mine = row0 + (int64_t)col * RPB;
  if (col < ROWS_PER_THREAD && r_mine < rows) {
    scale[r_mine] = s;
    zp[r_mine] = z;
  }
}

// One lane per 8 packed bytes: the high nibbles are elements col*8.., the low nibbles D/2 + col*8...
template <int D, bool F16>
__global__ __launch_bounds__(NTHREADS) void dequantize_rows4_kernel(const uint8_t* __restrict__ codes, const float* __restrict__ scale,
                                                                    const int32_t* __restrict__ zp, int64_t rows,
                                                                    uint16_t* __restrict__ out, int64_t out_row_stride) {
  constexpr int LPR = D / 16;
  const int64_t gid = (int64_t)blockIdx.x * NTHREADS + threadIdx.x;
  const int col = (int)(gid % LPR);
  const int64_t r = gid / LPR;
  if (r >= rows) return;
  const u32x2_t c = *(const u32x2_t*)(codes + r * (D / 2) + col * 8);
  const float s = scale[r];
  const int32_t z = zp[r];
  u32x4_t hi, lo;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t w = c[e >> 1] >> ((e & 1) * 16);
    hi[e] = dequant_pair<F16>((w >> 4) & 0xf, (w >> 12) & 0xf, z, s);
    lo[e] = dequant_pair<F16>(w & 0xf, (w >> 8) & 0xf, z, s);
  }
  *(u32x4_t*)(out + r * out_row_stride + col * 8) = hi;
  *(u32x4_t*)(out + r * out_row_stride + D / 2 + col * 8) = lo;
}

// ---- general blocks (several segments per block, 8 or 4 bits): one wavefront per block ------------

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fminf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

template <bool F16>
__device__ __forceinline__ u32x2_t codes_of_chunk(u32x4_t raw, float inv, float zf, float qmax) {
  u32x2_t out;
#pragma unroll
  for (int h = 0; h < 2; ++h)
    out[h] = quant_code(elem_lo<F16>(raw[2 * h]), inv, zf, qmax) | (quant_code(elem_hi<F16>(raw[2 * h]), inv, zf, qmax) << 8) |
             (quant_code(elem_lo<F16>(raw[2 * h + 1]), inv, zf, qmax) << 16) | (quant_code(elem_hi<F16>(raw[2 * h + 1]), inv, zf, qmax) << 24);
  return out;
}

template <int BITS, bool F16>
__global__ __launch_bounds__(NTHREADS) void quantize_blocks_kernel(const kvx_block_quant_args a) {
  const int lane = threadIdx.x & 63;
  const int64_t blk = (int64_t)blockIdx.x * (NTHREADS / 64) + (threadIdx.x >> 6);
  if (blk >= (int64_t)a.n_outer * a.n_inner) return;  // a whole wavefront at a time
  const int64_t outer = blk / a.n_inner, inner = blk % a.n_inner;
  const uint16_t* base = (const uint16_t*)a.x + outer * a.x_stride_outer + inner * a.x_stride_inner;
  const int cps = a.D / 8;  // chunks of 8 values per segment
  const int nchunks = a.nseg * cps;
  auto chunk = [&](int c) { return *(const u32x4_t*)(base + (int64_t)(c / cps) * a.x_stride_seg + (c % cps) * 8); };
  float mn = INFINITY, mx = -INFINITY, bad = 0.0f;
  for (int c = lane; c < nchunks; c += 64) {
    const u32x4_t raw = chunk(c);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mn = fminf(mn, fminf(elem_lo<F16>(raw[e]), elem_hi<F16>(raw[e])));
      mx = fmaxf(mx, fmaxf(elem_lo<F16>(raw[e]), elem_hi<F16>(raw[e])));
      bad = __builtin_isunordered(elem_lo<F16>(raw[e]), elem_hi<F16>(raw[e])) ? 1.0f : bad;
    }
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if (wave_max(bad) != 0.0f) mn = mx = __builtin_nanf("");  // as torch.aminmax: a NaN in the block is the block's extreme
  constexpr float qmax = BITS == 8 ? 255.0f : 15.0f;
  float s;
  int32_t z;
  quant_params(mn, mx, s, z, qmax);
  const float inv = 1.0f / s, zf = (float)z;
  uint8_t* out = a.codes + outer * a.codes_stride_outer + inner * ((int64_t)nchunks * BITS);  // nchunks * 8 values * BITS / 8 bytes
  if constexpr (BITS == 8) {
    for (int c = lane; c < nchunks; c += 64) *(u32x2_t*)(out + c * 8) = codes_of_chunk<F16>(chunk(c), inv, zf, qmax);
  } else {
    const int half = nchunks / 2;
    for (int c = lane; c < half; c += 64) {
      const u32x2_t hi = codes_of_chunk<F16>(chunk(c), inv, zf, qmax), lo = codes_of_chunk<F16>(chunk(c + half), inv, zf, qmax);
      *(u32x2_t*)(out + c * 8) = u32x2_t{(hi[0] << 4) | lo[0], (hi[1] << 4) | lo[1]};
    }
  }
  if (lane == 0) {
    a.scale[outer * a.state_stride_outer + inner] = s;
    a.zp[outer * a.state_stride_outer + inner] = z;
  }
}

template <int BITS, bool F16>
__global__ __launch_bounds__(NTHREADS) void dequantize_blocks_kernel(const kvx_block_quant_args a) {
  const int lane = threadIdx.x & 63;
  const int64_t blk = (int64_t)blockIdx.x * (NTHREADS / 64) + (threadIdx.x >> 6);
  if (blk >= (int64_t)a.n_outer * a.n_inner) return;
  const int64_t outer = blk / a.n_inner, inner = blk % a.n_inner;
  uint16_t* base = (uint16_t*)a.x + outer * a.x_stride_outer + inner * a.x_stride_inner;
  const int cps = a.D / 8;
  const int nchunks = a.nseg * cps;
  auto chunk_ptr = [&](int c) { return (u32x4_t*)(base + (int64_t)(c / cps) * a.x_stride_seg + (c % cps) * 8); };
  const float s = a.scale[outer * a.state_stride_outer + inner];
  const int32_t z = a.zp[outer * a.state_stride_outer + inner];
  const uint8_t* in = a.codes + outer * a.codes_stride_outer + inner * ((int64_t)nchunks * BITS);
  if constexpr (BITS == 8) {
    for (int c = lane; c < nchunks; c += 64) {
      const u32x2_t cc = *(const u32x2_t*)(in + c * 8);
      u32x4_t o;
      o[0] = dequant_pair<F16>(cc[0] & 0xff, (cc[0] >> 8) & 0xff, z, s);
      o[1] = dequant_pair<F16>((cc[0] >> 16) & 0xff, cc[0] >> 24, z, s);
      o[2] = dequant_pair<F16>(cc[1] & 0xff, (cc[1] >> 8) & 0xff, z, s);
      o[3] = dequant_pair<F16>((cc[1] >> 16) & 0xff, cc[1] >> 24, z, s);
      *chunk_ptr(c) = o;
    }
  } else {
    const int half = nchunks / 2;
    for (int c = lane; c < half; c += 64) {
      const u32x2_t cc = *(const u32x2_t*)(in + c * 8);
      u32x4_t hi, lo;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t w = cc[e >> 1] >> ((e & 1) * 16);
        hi[e] = dequant_pair<F16>((w >> 4) & 0xf, (w >> 12) & 0xf, z, s);
        lo[e] = dequant_pair<F16>(w & 0xf, (w >> 8) & 0xf, z, s);
      }
      *chunk_ptr(c) = hi;
      *chunk_ptr(c + half) = lo;
    }
  }
}

// Sum over the LPR adjacent lanes holding one row; every lane gets the result.
template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
  if constexpr (LPR >= 16)
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true));
  if constexpr (LPR == 32) v += __shfl_xor(v, 16, 64);  // the other DPP row of the group
  return v;
}

// |row|_2 of a bf16 (F16: fp16) row spread over LPR lanes, accumulated in fp32.
template <int LPR, bool F16 = false>
__device__ __forceinline__ float row_norm(u32x4_t raw) {
  float ss = 0.0f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float a = elem_lo<F16>(raw[e]), b = elem_hi<F16>(raw[e]);
    ss += a * a;
    ss += b * b;
  }
  return sqrtf(row_sum<LPR>(ss));
}

// |x - dq(q(x))|_2 of a row: the dequantised value and the difference are rounded to the rows' type, the norm
// accumulates in fp32 (keys_values/kvcache/quantize/pytorch.py:530-548).
template <int LPR, bool F16>
__device__ __forceinline__ float row_quant_error(u32x4_t raw, u32x2_t codes, float scale, int32_t zp) {
  float ss = 0.0f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t cw = codes[e >> 1];
    const int sh = (e & 1) * 16;
    const uint32_t dq = dequant_pair<F16>((cw >> sh) & 0xff, (cw >> (sh + 8)) & 0xff, zp, scale);
    const uint32_t diff = pack_pair<F16>(elem_lo<F16>(raw[e]) - elem_lo<F16>(dq), elem_hi<F16>(raw[e]) - elem_hi<F16>(dq));
    const float a = elem_lo<F16>(diff), b = elem_hi<F16>(diff);
    ss += a * a;
    ss += b * b;
  }
  return sqrtf(row_sum<LPR>(ss));
}

// One lane per 8 elements of one job (b, h, j), for K and V. Without a ring move job j writes new
// token j into index[b,h,j]. With one (j < grace_num) the lanes of the job first carry ring slot
// grace_slots[j] over to index[b,h,j], then write new token num - grace_num + j into the ring slot:
// the read and the write of that slot are issued by the same wavefront, in this order, and the
// read's data is consumed before the write is issued.
template <int D, int KV>
__global__ __launch_bounds__(NTHREADS) void cache_write_kernel(const kvx_cache_write_args a) {
  constexpr bool U8 = !kv_is_plain(KV);  // a quantised store: codes + row state
  constexpr bool U4 = kv_is_u4(KV);       // two codes per byte: only the lanes of the first half of a row store
  constexpr bool F16 = kv_elem_f16(KV);   // the rows are float16
  constexpr int LPR = D / 8;
  const int64_t gid = (int64_t)blockIdx.x * NTHREADS + threadIdx.x;
  const int col = (int)(gid % LPR);
  const int64_t rid = gid / LPR;
  const int64_t total = (int64_t)a.B * a.Hkv * a.num;
  const bool live = rid < total;
  const int64_t ridc = live ? rid : 0;
  const int j = (int)(ridc % a.num);
  const int hh = (int)((ridc / a.num) % a.Hkv);
  const int b = (int)(ridc / ((int64_t)a.num * a.Hkv));
  const int slot = a.index[b * a.index_stride_b + hh * a.index_stride_h + j];
  const bool moves = j < a.grace_num;
  const int ring = moves ? a.grace_slots[j] : -1;
  const int src = moves ? a.num - a.grace_num + j : j - a.grace_num;  // new token this job stores
  // a bad index is dropped, never written out of bounds
  const bool ok = live && slot >= 0 && slot < a.cache_len && (!moves || (ring >= 0 && ring < a.cache_len && ring != slot));
  const int wslot = moves ? ring : slot;  // where the new token goes
  const uint16_t* ks = (const uint16_t*)a.key + b * a.key_stride_b + hh * a.key_stride_h + (int64_t)src * a.key_stride_t + col * 8;
  const uint16_t* vs = (const uint16_t*)a.value + b * a.value_stride_b + hh * a.value_stride_h + (int64_t)src * a.value_stride_t + col * 8;
  const u32x4_t kr = live ? *(const u32x4_t*)ks : u32x4_t{0, 0, 0, 0};
  const u32x4_t vr = live ? *(const u32x4_t*)vs : u32x4_t{0, 0, 0, 0};
  const int64_t tp_row = b * a.tp_stride_b + hh * a.tp_stride_h;
  const int64_t sc_row = b * a.sc_stride_b + hh * a.sc_stride_h;
  const int64_t qs_row = b * a.qs_stride_b + hh * a.qs_stride_h;
  constexpr int ES = U8 ? 1 : 2;  // bytes per cache element
  const bool stores = !U4 || col < LPR / 2;
  const int ccol = U4 ? col % (LPR / 2) : col;
  uint8_t* kc_row = (uint8_t*)a.k_cache + (b * a.kc_stride_b + hh * a.kc_stride_h) * ES + ccol * 8 * ES;
  uint8_t* vc_row = (uint8_t*)a.v_cache + (b * a.vc_stride_b + hh * a.vc_stride_h) * ES + ccol * 8 * ES;

  // a quantised store: quantise the row held as (krow, vrow) by the LPR lanes of this job and store
  // it in slot `target`; every lane of the wavefront calls it (the row reductions need all lanes of a row)
  auto put = [&](const u32x4_t& krow, const u32x4_t& vrow, int target, bool doit, bool want_err) -> float {
    float s1, s2, err = 0.0f;
    int32_t z1, z2;
    u32x2_t kc = U4 ? quantize4<LPR, F16>(krow, s1, z1) : quantize8<LPR, F16>(krow, s1, z1);
    u32x2_t vc = U4 ? quantize4<LPR, F16>(vrow, s2, z2) : quantize8<LPR, F16>(vrow, s2, z2);
    if (want_err) err = row_quant_error<LPR, F16>(krow, kc, s1, z1) + row_quant_error<LPR, F16>(vrow, vc, s2, z2);  // uniform branch
    if constexpr (U4) {  // byte j = code[j] << 4 | code[j + D/2]: the partner lane holds the low nibbles
      kc = u32x2_t{(kc[0] << 4) | (uint32_t)__shfl_xor(kc[0], LPR / 2, 64), (kc[1] << 4) | (uint32_t)__shfl_xor(kc[1], LPR / 2, 64)};
      vc = u32x2_t{(vc[0] << 4) | (uint32_t)__shfl_xor(vc[0], LPR / 2, 64), (vc[1] << 4) | (uint32_t)__shfl_xor(vc[1], LPR / 2, 64)};
    }
    if (doit) {
      if (stores) {
        *(u32x2_t*)(kc_row + (int64_t)target * a.kc_stride_t) = kc;
        *(u32x2_t*)(vc_row + (int64_t)target * a.vc_stride_t) = vc;
      }
      if (col == 0) {
        a.k_scale[qs_row + target] = s1;
        a.k_zp[qs_row + target] = z1;
        a.v_scale[qs_row + target] = s2;
        a.v_zp[qs_row + target] = z2;
      }
    }
    return err;
  };

  if (a.grace_num > 0) {  // uniform over the launch
    const bool mv = ok && moves;
    if constexpr (!U8) {
      if (mv) {
        *(u32x4_t*)(kc_row + (int64_t)slot * a.kc_stride_t * ES) = *(const u32x4_t*)(kc_row + (int64_t)ring * a.kc_stride_t * ES);
        *(u32x4_t*)(vc_row + (int64_t)slot * a.vc_stride_t * ES) = *(const u32x4_t*)(vc_row + (int64_t)ring * a.vc_stride_t * ES);
      }
    } else {
      // The moved row is written like any other: its dequantised values are quantised again
      // (keys_values/kvcache/attn_weights.py:578-590 reads the ring rows from the dequantised buffer
      // and hands them to the same write as the new rows), which is not the identity on the codes.
      u32x4_t krow = {0, 0, 0, 0}, vrow = {0, 0, 0, 0};
      if (mv) {
        u32x2_t kq = *(const u32x2_t*)(kc_row + (int64_t)ring * a.kc_stride_t);
        u32x2_t vq = *(const u32x2_t*)(vc_row + (int64_t)ring * a.vc_stride_t);
        if constexpr (U4) {
          kq = u4_codes(kq, col < LPR / 2 ? 4 : 0);
          vq = u4_codes(vq, col < LPR / 2 ? 4 : 0);
        }
        krow = dequant_words<F16>(kq[0], kq[1], a.k_zp[qs_row + ring], a.k_scale[qs_row + ring]);
        vrow = dequant_words<F16>(vq[0], vq[1], a.v_zp[qs_row + ring], a.v_scale[qs_row + ring]);
      }
      put(krow, vrow, slot, mv, false);
    }
    if (mv && col == 0) {
      if (a.token_pos) a.token_pos[tp_row + slot] = a.input_pos - a.grace_period + j;
      if (a.scores) a.scores[sc_row + slot] = a.scores[sc_row + ring];
      if (a.v_norm) a.v_norm[sc_row + slot] = a.v_norm[sc_row + ring];
      if (a.q_errors) a.q_errors[sc_row + slot] = a.q_errors[sc_row + ring];
    }
  }

  float qerr = 0.0f;
  if constexpr (!U8) {
    if (ok) {
      *(u32x4_t*)(kc_row + (int64_t)wslot * a.kc_stride_t * ES) = kr;
      *(u32x4_t*)(vc_row + (int64_t)wslot * a.vc_stride_t * ES) = vr;
    }
  } else {
    qerr = put(kr, vr, wslot, ok, a.q_errors != nullptr);
  }
  float vnorm = 0.0f;
  if (a.v_norm) vnorm = row_norm<LPR, F16>(vr);  // uniform branch: every lane takes part in the reduction
  if (live && col == 0 && a.replay_log) {  // the slot as consumed, valid or not: the log mirrors index
    const int64_t lp = a.log_pos + j;
    a.replay_log[(lp / a.log_blocksize) * a.log_stride_block + b * a.log_stride_b + hh * a.log_stride_h + lp % a.log_blocksize] =
        (uint32_t)slot;
  }
  if (ok && col == 0) {
    if (a.token_pos) a.token_pos[tp_row + wslot] = a.input_pos + src;
    if (a.scores) a.scores[sc_row + wslot] = 0.0f;
    if (a.v_norm) a.v_norm[sc_row + wslot] = vnorm;
    if (a.q_errors) a.q_errors[sc_row + wslot] = qerr;
  }
}

}  // namespace

// D in {64, 128, 256}, bits in {8, 4}, f16: the rows are float16 (else bfloat16)
template <int D, bool F16>
int launch_quantize_rows_t(const void* x, int64_t x_row_stride, int64_t rows, int bits, uint8_t* codes, float* scale, int32_t* zp, hipStream_t st) {
  const int rpb = (NTHREADS / (D / 8)) * ROWS_PER_THREAD;
  const unsigned grid = (unsigned)((rows + rpb - 1) / rpb);
  if (bits == 8) hipLaunchKernelGGL((quantize_rows_kernel<D, F16>), dim3(grid), dim3(NTHREADS), 0, st, (const uint16_t*)x, x_row_stride, rows, codes, scale, zp);
  else hipLaunchKernelGGL((quantize_rows4_kernel<D, F16>), dim3(grid), dim3(NTHREADS), 0, st, (const uint16_t*)x, x_row_stride, rows, codes, scale, zp);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

int launch_quantize_rows(const void* x, int64_t x_row_stride, int64_t rows, int D, int bits, bool f16, uint8_t* codes, float* scale,
                         int32_t* zp, hipStream_t st) {
  if (rows == 0) return KVX_OK;
  if (D == 256) return f16 ? launch_quantize_rows_t<256, true>(x, x_row_stride, rows, bits, codes, scale, zp, st)
                           : launch_quantize_rows_t<256, false>(x, x_row_stride, rows, bits, codes, scale, zp, st);
  if (D == 128) return f16 ? launch_quantize_rows_t<128, true>(x, x_row_stride, rows, bits, codes, scale, zp, st)
                           : launch_quantize_rows_t<128, false>(x, x_row_stride, rows, bits, codes, scale, zp, st);
  return f16 ? launch_quantize_rows_t<64, true>(x, x_row_stride, rows, bits, codes, scale, zp, st)
             : launch_quantize_rows_t<64, false>(x, x_row_stride, rows, bits, codes, scale, zp, st);
}

template <int D, bool F16>
int launch_dequantize_rows_t(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int bits, void* out,
                             int64_t out_row_stride, hipStream_t st) {
  if (bits == 8) {
    const int rpb = (NTHREADS / (D / 8)) * ROWS_PER_THREAD;
    const unsigned grid = (unsigned)((rows + rpb - 1) / rpb);
    hipLaunchKernelGGL((dequantize_rows_kernel<D, F16>), dim3(grid), dim3(NTHREADS), 0, st, codes, scale, zp, rows, (uint16_t*)out, out_row_stride);
  } else {
    const int64_t lanes = rows * (D / 16);
    const unsigned grid = (unsigned)((lanes + NTHREADS - 1) / NTHREADS);
    hipLaunchKernelGGL((dequantize_rows4_kernel<D, F16>), dim3(grid), dim3(NTHREADS), 0, st, codes, scale, zp, rows, (uint16_t*)out, out_row_stride);
  }
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

int launch_dequantize_rows(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int D, int bits, bool f16,
                           void* out, int64_t out_row_stride, hipStream_t st) {
  if (rows == 0) return KVX_OK;
  if (D == 256) return f16 ? launch_dequantize_rows_t<256, true>(codes, scale, zp, rows, bits, out, out_row_stride, st)
                           : launch_dequantize_rows_t<256, false>(codes, scale, zp, rows, bits, out, out_row_stride, st);
  if (D == 128) return f16 ? launch_dequantize_rows_t<128, true>(codes, scale, zp, rows, bits, out, out_row_stride, st)
                           : launch_dequantize_rows_t<128, false>(codes, scale, zp, rows, bits, out, out_row_stride, st);
  return f16 ? launch_dequantize_rows_t<64, true>(codes, scale, zp, rows, bits, out, out_row_stride, st)
             : launch_dequantize_rows_t<64, false>(codes, scale, zp, rows, bits, out, out_row_stride, st);
}

int launch_quantize_blocks(const kvx_block_quant_args& a, hipStream_t st) {
  const int64_t blocks = (int64_t)a.n_outer * a.n_inner;
  if (blocks == 0) return KVX_OK;
  const unsigned grid = (unsigned)((blocks + NTHREADS / 64 - 1) / (NTHREADS / 64));
  const bool f16 = a.elem_dtype == KVX_KV_F16;
  if (a.bits == 8 && f16) hipLaunchKernelGGL((quantize_blocks_kernel<8, true>), dim3(grid), dim3(NTHREADS), 0, st, a);
  else if (a.bits == 8) hipLaunchKernelGGL((quantize_blocks_kernel<8, false>), dim3(grid), dim3(NTHREADS), 0, st, a);
  else if (f16) hipLaunchKernelGGL((quantize_blocks_kernel<4, true>), dim3(grid), dim3(NTHREADS), 0, st, a);
  else hipLaunchKernelGGL((quantize_blocks_kernel<4, false>), dim3(grid), dim3(NTHREADS), 0, st, a);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

int launch_dequantize_blocks(const kvx_block_quant_args& a, hipStream_t st) {
  const int64_t blocks = (int64_t)a.n_outer * a.n_inner;
  if (blocks == 0) return KVX_OK;
  const unsigned grid = (unsigned)((blocks + NTHREADS / 64 - 1) / (NTHREADS / 64));
  const bool f16 = a.elem_dtype == KVX_KV_F16;
  if (a.bits == 8 && f16) hipLaunchKernelGGL((dequantize_blocks_kernel<8, true>), dim3(grid), dim3(NTHREADS), 0, st, a);
  else if (a.bits == 8) hipLaunchKernelGGL((dequantize_blocks_kernel<8, false>), dim3(grid), dim3(NTHREADS), 0, st, a);
  else if (f16) hipLaunchKernelGGL((dequantize_blocks_kernel<4, true>), dim3(grid), dim3(NTHREADS), 0, st, a);
  else hipLaunchKernelGGL((dequantize_blocks_kernel<4, false>), dim3(grid), dim3(NTHREADS), 0, st, a);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

template <int D>
int launch_cache_write_d(const kvx_cache_write_args& a, unsigned grid, hipStream_t st) {
  switch (a.kv_dtype) {
    case KVX_KV_F16: hipLaunchKernelGGL((cache_write_kernel<D, KVX_KV_F16>), dim3(grid), dim3(NTHREADS), 0, st, a); break;
    case KVX_KV_BF16: hipLaunchKernelGGL((cache_write_kernel<D, KVX_KV_BF16>), dim3(grid), dim3(NTHREADS), 0, st, a); break;
    case KVX_KV_U4: hipLaunchKernelGGL((cache_write_kernel<D, KVX_KV_U4>), dim3(grid), dim3(NTHREADS), 0, st, a); break;
    case KVX_KV_U8: hipLaunchKernelGGL((cache_write_kernel<D, KVX_KV_U8>), dim3(grid), dim3(NTHREADS), 0, st, a); break;
    case KVX_KV_U4_F16: hipLaunchKernelGGL((cache_write_kernel<D, KVX_KV_U4_F16>), dim3(grid), dim3(NTHREADS), 0, st, a); break;
    default: hipLaunchKernelGGL((cache_write_kernel<D, KVX_KV_U8_F16>), dim3(grid), dim3(NTHREADS), 0, st, a); break;
  }
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

int launch_cache_write(const kvx_cache_write_args& a, hipStream_t st) {
  const int64_t total = (int64_t)a.B * a.Hkv * a.num * (a.D / 8);
  if (total == 0) return KVX_OK;
  const unsigned grid = (unsigned)((total + NTHREADS - 1) / NTHREADS);
  if (a.D == 256) return launch_cache_write_d<256>(a, grid, st);
  if (a.D == 128) return launch_cache_write_d<128>(a, grid, st);
  return launch_cache_write_d<64>(a, grid, st);
}

}  // namespace kvx
