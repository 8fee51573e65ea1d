// Shared device/host helpers for the libkvx kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <limits.h>

#include "../../include/kvx.h"

// The kernels are written for gfx950 alone: its matrix instructions and transposing LDS reads, the direct
// global -> LDS transfers, and (decode) cross-workgroup hand-offs through device-scope relaxed atomics that rely on
// what this hardware does -- such stores write through to memory shared by all its dies and are counted by vmcnt,
// such loads do not hit in the per-CU cache. Another target has to revisit all of that.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "libkvx: device code must be compiled with --offload-arch=gfx950 only"
#endif

namespace kvx {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kWave = 64;

// Records the message kvx_last_error() returns on this thread, returns `code`.
int set_error(int code, const char* fmt, ...);
int hip_error(hipError_t e, const char* what);

#define KVX_REQUIRE(cond, code, ...)            \
  do {                                          \
    if (!(cond)) return ::kvx::set_error((code), __VA_ARGS__); \
  } while (0)

#define KVX_HIP(call)                                      \
  do {                                                     \
    hipError_t e__ = (call);                               \
    if (e__ != hipSuccess) return ::kvx::hip_error(e__, #call); \
  } while (0)

// ---- launchers implemented one per translation unit ---------------------------------------
int launch_sdpa_prefill(const kvx_sdpa_args& a, hipStream_t st);
size_t sdpa_prefill_workspace(const kvx_sdpa_args& a);
int launch_score_sum(const kvx_sdpa_args& a, hipStream_t st);
size_t score_sum_workspace(const kvx_sdpa_args& a);
int launch_sdpa_decode(const kvx_sdpa_args& a, const kvx_h2o_args* fused_h2o, hipStream_t st);
size_t sdpa_decode_workspace(const kvx_sdpa_args& a, bool fused_h2o);
void set_decode_tuning(int resident, int spin_limit, int poll_sleep);
int launch_quantize_rows(const void* x, int64_t x_row_stride, int64_t rows, int D, int bits, bool f16, uint8_t* codes, float* scale,
                         int32_t* zp, hipStream_t st);
int launch_dequantize_rows(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int D, int bits, bool f16, void* out,
                           int64_t out_row_stride, hipStream_t st);
int launch_quantize_blocks(const kvx_block_quant_args& a, hipStream_t st);
int launch_dequantize_blocks(const kvx_block_quant_args& a, hipStream_t st);
int launch_cache_write(const kvx_cache_write_args& a, hipStream_t st);
int launch_h2o_update_select(const kvx_h2o_args& a, hipStream_t st);
size_t h2o_workspace(const kvx_h2o_args& a);
int launch_h2o_update_select_static(const kvx_h2o_args& a, hipStream_t st);
size_t h2o_static_scratch_bytes();
int launch_rmsnorm_rows(const void* x, int64_t x_rs, void* out, int64_t o_rs, const float* weight, int64_t rows, int dim, float eps,
                        hipStream_t st);
int launch_add_rmsnorm_rows(const void* x, int64_t x_rs, const void* delta, int64_t d_rs, void* x_out, int64_t xo_rs, void* out,
                            int64_t o_rs, const float* weight, int64_t rows, int dim, float eps, hipStream_t st);
int launch_swiglu_rows(const void* gate_up, int64_t g_rs, void* out, int64_t o_rs, int64_t rows, int dim, hipStream_t st);
int launch_qk_norm_rope(void* qkv, int64_t sb, int64_t stt, int B, int num, int Hq, int Hkv, int D, const float* qw, const float* kw,
                        float eps, const float* cos_t, const float* sin_t, int input_pos, hipStream_t st);

// Number of compute units of the current device (cached).
int num_cus();

// ---- device helpers ------------------------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// Round-to-nearest-even fp32 -> bf16 (two at a time), bit pattern in a dword (lo = a, hi = b).
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2_t r = __builtin_convertvector(f32x2_t{a, b}, bf16x2_t);
  return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ bf16x8_t as_bf16x8(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }

// ---- the two 16-bit element types of q / k / v / o: bf16 and, with KVX_KV_F16, fp16 -----------------
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

// plain rows of the query's own type (no codes)
constexpr bool kv_is_plain(int kv) { return kv == KVX_KV_BF16 || kv == KVX_KV_F16; }
// q, o and the (dequantised) rows are float16, else bfloat16
constexpr bool kv_elem_f16(int kv) { return kv == KVX_KV_F16 || kv == KVX_KV_U8_F16 || kv == KVX_KV_U4_F16; }
// two codes per byte
constexpr bool kv_is_u4(int kv) { return kv == KVX_KV_U4 || kv == KVX_KV_U4_F16; }
constexpr bool kv_valid(int kv) { return kv >= KVX_KV_BF16 && kv <= KVX_KV_U4_F16; }

// the two halves of a packed pair of the element type as fp32
template <bool F16>
__device__ __forceinline__ float elem_lo(uint32_t packed) {
  if constexpr (F16) return (float)__builtin_bit_cast(f16x2_t, packed)[0];
  else return __uint_as_float(packed << 16);
}
template <bool F16>
__device__ __forceinline__ float elem_hi(uint32_t packed) {
  if constexpr (F16) return (float)__builtin_bit_cast(f16x2_t, packed)[1];
  else return __uint_as_float(packed & 0xffff0000u);
}

// D = A B + C on one 32x32x16 tile, operands as four dwords of eight 16-bit values
template <bool F16>
__device__ __forceinline__ f32x16_t mfma_32x32x16(u32x4_t a, u32x4_t b, f32x16_t c) {
  if constexpr (F16) return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// two fp32 -> packed pair of the element type, round to nearest even (lo = a, hi = b)
template <bool F16>
__device__ __forceinline__ uint32_t pack_pair(float a, float b) {
  if constexpr (F16) {
    // two scalar conversions (round to nearest even): a conversion of the pair as a vector trips the instruction
    // selector when packed fp32 arithmetic is switched off and one operand is a negation
    const f16x2_t r = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, r);
  } else {
    return pack_bf16(a, b);
  }
}

// acc + x.lo * y.lo + x.hi * y.hi on packed pairs of the element type
template <bool F16>
__device__ __forceinline__ float dot2_acc(uint32_t x, uint32_t y, float acc) {
  if constexpr (F16) return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, x), __builtin_bit_cast(f16x2_t, y), acc, false);
  else return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, x), __builtin_bit_cast(bf16x2_t, y), acc, false);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Exchange with the lane 32 away (the other half of the wavefront).
__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

// max / sum of a value with the lane 32 away, in every lane, through v_permlane32_swap (a vector ALU
// exchange of the two wavefront halves; no LDS round trip as with a shuffle).
typedef uint32_t u32pair_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float max_halves(float v) {
  const u32pair_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_halves(float v) {
  const u32pair_t r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The affine 8-bit row quantiser, one element. `inv` = 1.0f / scale, `zf` = (float) zero point.
// rint before the add, so the multiply can never fuse with it.
// `qmax` = 255 (8-bit) or 15 (4-bit codes).
__device__ __forceinline__ uint32_t quant_code(float x, float inv, float zf, float qmax = 255.0f) {
  float c = __builtin_rintf(x * inv) + zf;
  c = fminf(fmaxf(c, 0.0f), qmax);
  return (uint32_t)c;
}

// scale and zero point of a row from its min and max (IEEE division, no fast-math).
__device__ __forceinline__ void quant_params(float mn, float mx, float& scale, int32_t& zp, float qmax = 255.0f) {
  float s = (mx - mn) / qmax;
  s = s < 1.1920929e-07f ? 1.1920929e-07f : s;  // torch.clamp(min=eps): a NaN stays a NaN (fmaxf would drop it)
  scale = s;
  zp = 0 - (int32_t)__builtin_rintf(mn / s);
}

// elem( (float)((int)code - zp) * scale ), two codes -> packed dword of the element type (bf16, or fp16 with F16).
template <bool F16 = false>
__device__ __forceinline__ uint32_t dequant_pair(uint32_t c0, uint32_t c1, int32_t zp, float scale) {
  float a = (float)((int32_t)c0 - zp) * scale;
  float b = (float)((int32_t)c1 - zp) * scale;
  return pack_pair<F16>(a, b);
}

// 8 byte-sized codes (two dwords) -> 8 values of the element type (four dwords). (Forming code - zp in fp32 from
// byte-to-float conversions is exact for |zp| < 2^24 but measured no faster than this integer form; forming it
// in packed fp16 (bytes 0x64, code = 1024 + code; v_pk_add_f16 of -(1024 + zp); v_fma_mix_f32 by the scale) gives
// the same bits with one instruction less per value for small zero points and measured 5 - 7 % slower in the
// decode and prefill kernels.)
template <bool F16 = false>
__device__ __forceinline__ u32x4_t dequant_words(uint32_t c0, uint32_t c1, int32_t zp, float scale) {
  u32x4_t r;
  r[0] = dequant_pair<F16>(c0 & 0xff, (c0 >> 8) & 0xff, zp, scale);
  r[1] = dequant_pair<F16>((c0 >> 16) & 0xff, c0 >> 24, zp, scale);
  r[2] = dequant_pair<F16>(c1 & 0xff, (c1 >> 8) & 0xff, zp, scale);
  r[3] = dequant_pair<F16>((c1 >> 16) & 0xff, c1 >> 24, zp, scale);
  return r;
}

// 4-bit store (two codes per byte, first half of the row in the high nibbles): chunk c (values
// 8c .. 8c+7) of a row of D values lies in one nibble of the 8 bytes at u4_byte_off, and becomes 8
// byte-sized codes with u4_codes.
template <int D>
__device__ __forceinline__ uint32_t u4_byte_off(int c) { return (uint32_t)(c % (D / 16)) * 8u; }
template <int D>
__device__ __forceinline__ int u4_shift(int c) { return c < D / 16 ? 4 : 0; }
__device__ __forceinline__ u32x2_t u4_codes(u32x2_t bytes, int shift) {
  return u32x2_t{(bytes[0] >> shift) & 0x0f0f0f0fu, (bytes[1] >> shift) & 0x0f0f0f0fu};
}

// ---- global -> LDS transfers without registers ----------------------------------------------------------------

// 16 bytes per lane straight from global memory into LDS (global_load_lds_dwordx4): lane l lands at
// lds_addr + 16 l, lds_addr uniform over the wavefront. Written as inline assembly so that the
// compiler does not serialise later LDS reads of OTHER buffers behind the transfer; the kernel
// waits for its transfers itself (s_waitcnt vmcnt(0)) before the barrier that publishes a tile.
__device__ __forceinline__ void dma16(const char* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(base)
               : "memory", "m0");
}
// the same with the LDS address formed as lds_base + IMM in M0 by the one scalar instruction the
// transfer needs anyway
template <uint32_t IMM>
__device__ __forceinline__ void dma16_at(const char* base, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_base), "v"(voff), "s"(base), "n"(IMM)
               : "memory", "m0", "scc");
}
// same for 4 bytes per lane (global_load_lds_dword): lane l lands at lds_addr + 4 l
__device__ __forceinline__ void dma4(const char* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_addr), "v"(voff), "s"(base)
               : "memory", "m0");
}
template <uint32_t IMM>
__device__ __forceinline__ void dma4_at(const char* base, uint32_t voff, uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(lds_base), "v"(voff), "s"(base), "n"(IMM)
               : "memory", "m0", "scc");
}
__device__ __forceinline__ uint32_t lds_addr_of(const void* p) {
  return (uint32_t)(uintptr_t)((const __attribute__((address_space(3))) char*)p);
}


}  // namespace kvx
