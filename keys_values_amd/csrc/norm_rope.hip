// RMS normalisation of rows, and the per-head query/key normalisation fused with the rotary position
// encoding, for gfx950 (both HBM-bound, one pass).
//
// Reference behaviour:
//   RMSNorm.forward, keys_values/model.py:870-878: x32 = float(x); n = |x32|_2 / sqrt(size);
//     y = (x32 / (n + eps)) * weight, cast to the input type. eps is added to the norm, not under the
//     root, and the division happens before the multiplication by the weight.
//   CausalSelfAttention.forward, keys_values/model.py:733-775: q and k are normalised per head over
//     head_size (norm_q / norm_k), cast back to bf16, then rotated (apply_rope,
//     keys_values/pos_encoding.py:34-44 -> y = x * cos + cat(-x2, x1) * sin in fp32, half-split
//     convention, keys_values/fused/fused_rope.py:57-87,198-200) and cast to bf16 again.
// The fused kernel keeps both casts, so it returns what the two separate steps return. It works in
// place on the output of the QKV projection, (B, num, (Hq + 2 Hkv) * D): the value heads are left as
// they are and no transposed copies are made (the attention and cache kernels take strides).
#include "kvx_common.h"

namespace kvx {
namespace {

constexpr int NT = 256;

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
  return x;
}

// Sum over the WPR wavefronts that share a row (WPR = 1: the wavefront's own sum; WPR = NT / 64: the
// whole workgroup, through LDS, added in wavefront order).
template <int WPR>
__device__ __forceinline__ float row_total(float ss) {
  ss = wave_sum(ss);
  if constexpr (WPR > 1) {
    static_assert(WPR == NT / 64, "a row is one wavefront or the whole workgroup");
    __shared__ float part[WPR];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = part[0];
#pragma unroll
    for (int i = 1; i < WPR; ++i) ss += part[i];
  }
  return ss;
}

// WPR wavefronts per row; a lane holds up to MAXC chunks of 8 elements (dim <= 64 * WPR * 8 * MAXC).
// Few long rows (a 1024-token chunk of hidden states) take the whole workgroup per row: four times the
// loads in flight per row, and enough workgroups to cover the chip.
template <int MAXC, int WPR>
__global__ __launch_bounds__(NT) void rmsnorm_rows_kernel(const uint16_t* __restrict__ x, int64_t x_rs, uint16_t* __restrict__ out,
                                                          int64_t o_rs, const float* __restrict__ weight, int64_t rows, int dim,
                                                          float eps, float factor) {
  constexpr int TPR = 64 * WPR;  // threads per row
  const int lane = threadIdx.x % TPR;
  const int64_t row = (int64_t)blockIdx.x * (NT / TPR) + threadIdx.x / TPR;
  if (row >= rows) return;  // uniform over the threads of a row (and over the workgroup when WPR > 1)
  const int nchunks = dim / 8;
  const uint16_t* xr = x + row * x_rs;
  u32x4_t v[MAXC];
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = lane + TPR * c;
    v[c] = u32x4_t{0, 0, 0, 0};
    if (ch < nchunks) v[c] = *(const u32x4_t*)(xr + ch * 8);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float a = bf16_lo(v[c][e]), b = bf16_hi(v[c][e]);
      ss += a * a;
      ss += b * b;
    }
  }
  ss = row_total<WPR>(ss);
  const float denom = sqrtf(ss) * factor + eps;
  uint16_t* orow = out + row * o_rs;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = lane + TPR * c;
    if (ch >= nchunks) break;
    const f32x4_t w0 = *(const f32x4_t*)(weight + ch * 8);
    const f32x4_t w1 = *(const f32x4_t*)(weight + ch * 8 + 4);
    u32x4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float wa = e < 2 ? w0[2 * e] : w1[2 * e - 4];
      const float wb = e < 2 ? w0[2 * e + 1] : w1[2 * e - 3];
      o[e] = pack_bf16((bf16_lo(v[c][e]) / denom) * wa, (bf16_hi(v[c][e]) / denom) * wb);
    }
    *(u32x4_t*)(orow + ch * 8) = o;
  }
}

// x_out = bf16(x + delta) and out = RMSNorm(x_out) in one pass: the residual add of a block fused with
// the normalisation that follows it (keys_values/model.py:560-584: x = attention_output + x, then
// norm_2(x); x = mlp_output + x, then the next block's norm_1). The sum is rounded to bf16 before it is
// normalised, as the two separate steps do. In place is allowed (x_out == x).
template <int MAXC, int WPR>
__global__ __launch_bounds__(NT) void add_rmsnorm_rows_kernel(const uint16_t* x, int64_t x_rs, const uint16_t* __restrict__ delta,
                                                              int64_t d_rs, uint16_t* x_out, int64_t xo_rs,
                                                              uint16_t* __restrict__ out, int64_t o_rs, const float* __restrict__ weight,
                                                              int64_t rows, int dim, float eps, float factor) {
  constexpr int TPR = 64 * WPR;
  const int lane = threadIdx.x % TPR;
  const int64_t row = (int64_t)blockIdx.x * (NT / TPR) + threadIdx.x / TPR;
  if (row >= rows) return;
  const int nchunks = dim / 8;
  u32x4_t v[MAXC];
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = lane + TPR * c;
    v[c] = u32x4_t{0, 0, 0, 0};
    if (ch < nchunks) {
      const u32x4_t a = *(const u32x4_t*)(x + row * x_rs + ch * 8);
      const u32x4_t b = *(const u32x4_t*)(delta + row * d_rs + ch * 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[c][e] = pack_bf16(bf16_lo(a[e]) + bf16_lo(b[e]), bf16_hi(a[e]) + bf16_hi(b[e]));
      *(u32x4_t*)(x_out + row * xo_rs + ch * 8) = v[c];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float a = bf16_lo(v[c][e]), b = bf16_hi(v[c][e]);
      ss += a * a;
      ss += b * b;
    }
  }
  ss = row_total<WPR>(ss);
  const float denom = sqrtf(ss) * factor + eps;
  uint16_t* orow = out + row * o_rs;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = lane + TPR * c;
    if (ch >= nchunks) break;
    const f32x4_t w0 = *(const f32x4_t*)(weight + ch * 8);
    const f32x4_t w1 = *(const f32x4_t*)(weight + ch * 8 + 4);
    u32x4_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float wa = e < 2 ? w0[2 * e] : w1[2 * e - 4];
      const float wb = e < 2 ? w0[2 * e + 1] : w1[2 * e - 3];
      o[e] = pack_bf16((bf16_lo(v[c][e]) / denom) * wa, (bf16_hi(v[c][e]) / denom) * wb);
    }
    *(u32x4_t*)(orow + ch * 8) = o;
  }
}

// out[r, j] = bf16( bf16(silu(g[r, j])) * u[r, j] ), g = gate_up[r, j], u = gate_up[r, dim + j]: the
// gated activation of LLaMAMLP (proj(silu(fc_1 x) * fc_2 x)) on the output of one GEMM over the stacked
// fc_1 / fc_2 weights. silu is x / (1 + exp(-x)) in fp32, rounded to bf16 before the product, as the
// two separate tensor operations round.
__global__ __launch_bounds__(NT) void swiglu_rows_kernel(const uint16_t* __restrict__ gate_up, int64_t g_rs, uint16_t* __restrict__ out,
                                                         int64_t o_rs, int64_t rows, int dim) {
  const int cpr = dim / 8;
  const int64_t gid = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (gid >= rows * cpr) return;
  const int64_t r = gid / cpr;
  const int c = (int)(gid % cpr);
  const u32x4_t g = *(const u32x4_t*)(gate_up + r * g_rs + c * 8);
  const u32x4_t u = *(const u32x4_t*)(gate_up + r * g_rs + dim + c * 8);
  u32x4_t o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float g0 = bf16_lo(g[e]), g1 = bf16_hi(g[e]);
    const uint32_t act = pack_bf16(g0 / (1.0f + expf(-g0)), g1 / (1.0f + expf(-g1)));
    o[e] = pack_bf16(bf16_lo(act) * bf16_lo(u[e]), bf16_hi(act) * bf16_hi(u[e]));
  }
  *(u32x4_t*)(out + r * o_rs + c * 8) = o;
}

// One lane per 8 elements of a head row; LPR = D / 8 lanes share a row. Rows are (b, t, head) with
// head in [0, Hq + Hkv): the query heads, then the key heads, of token t.
template <int D>
__global__ __launch_bounds__(NT) void qk_norm_rope_kernel(uint16_t* __restrict__ qkv, int64_t sb, int64_t st, int B, int num, int Hq,
                                                          int Hkv, const float* __restrict__ qw, const float* __restrict__ kw,
                                                          float eps, float factor, const float* __restrict__ cos_t,
                                                          const float* __restrict__ sin_t, int input_pos) {
  constexpr int LPR = D / 8;
  constexpr int HALF = D / 2;
  const int col = threadIdx.x % LPR;
  const int64_t rid = (int64_t)blockIdx.x * (NT / LPR) + threadIdx.x / LPR;
  const int heads = Hq + Hkv;
  const int64_t total = (int64_t)B * num * heads;
  const bool live = rid < total;
  const int64_t r = live ? rid : 0;  // dead lanes follow row 0 so that the shuffles below stay defined
  const int head = (int)(r % heads);
  const int t = (int)((r / heads) % num);
  const int b = (int)(r / ((int64_t)heads * num));
  uint16_t* p = qkv + b * sb + (int64_t)t * st + (int64_t)head * D + col * 8;
  const u32x4_t raw = *(const u32x4_t*)p;
  float y[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    y[2 * e] = bf16_lo(raw[e]);
    y[2 * e + 1] = bf16_hi(raw[e]);
  }
  const float* w = head < Hq ? qw : kw;
  if (w) {  // uniform: either both weights are given or none
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += y[e] * y[e];
#pragma unroll
    for (int off = 1; off < LPR; off <<= 1) ss += __shfl_xor(ss, off, 64);
    const float denom = sqrtf(ss) * factor + eps;
    const f32x4_t w0 = *(const f32x4_t*)(w + col * 8);
    const f32x4_t w1 = *(const f32x4_t*)(w + col * 8 + 4);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float wv = e < 4 ? w0[e] : w1[e - 4];
      // the reference casts the normalised head back to bf16 before it is rotated
      y[e] = bf16_bits_to_f32(pack_bf16((y[e] / denom) * wv, 0.0f) & 0xffffu);
    }
  }
  // rotation: element d pairs with d +- D/2, held by the lane LPR/2 away; first half gets -x2, second +x1
  const bool first = col < LPR / 2;
  const int j0 = (col * 8) % HALF;
  const float* cr = cos_t + (int64_t)(input_pos + t) * HALF + j0;
  const float* sr = sin_t + (int64_t)(input_pos + t) * HALF + j0;
  const f32x4_t c0 = *(const f32x4_t*)cr, c1 = *(const f32x4_t*)(cr + 4);
  const f32x4_t s0 = *(const f32x4_t*)sr, s1 = *(const f32x4_t*)(sr + 4);
  u32x4_t o;
  float res[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float other = __shfl_xor(y[e], LPR / 2, 64);
    const float rot = first ? -other : other;
    const float cv = e < 4 ? c0[e] : c1[e - 4];
    const float sv = e < 4 ? s0[e] : s1[e - 4];
    res[e] = y[e] * cv + rot * sv;
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = pack_bf16(res[2 * e], res[2 * e + 1]);
  if (live) *(u32x4_t*)p = o;
}

// Rows of at least 2048 values, too few of them to fill the chip with a wavefront each.
bool workgroup_per_row(int64_t rows, int dim) { return dim >= 2048 && dim <= NT * 8 * 4 && rows <= 16384; }

}  // namespace

int launch_rmsnorm_rows(const void* x, int64_t x_rs, void* out, int64_t o_rs, const float* weight, int64_t rows, int dim, float eps,
                        hipStream_t st) {
  if (rows == 0) return KVX_OK;
  const float factor = 1.0f / sqrtf((float)dim);
  const unsigned grid = (unsigned)((rows + NT / 64 - 1) / (NT / 64));
  const int chunks_per_lane = (dim / 8 + 63) / 64;
  if (workgroup_per_row(rows, dim))
    hipLaunchKernelGGL((rmsnorm_rows_kernel<4, NT / 64>), dim3((unsigned)rows), dim3(NT), 0, st, (const uint16_t*)x, x_rs, (uint16_t*)out, o_rs,
                       weight, rows, dim, eps, factor);
  else if (chunks_per_lane <= 4)
    hipLaunchKernelGGL((rmsnorm_rows_kernel<4, 1>), dim3(grid), dim3(NT), 0, st, (const uint16_t*)x, x_rs, (uint16_t*)out, o_rs, weight, rows,
                       dim, eps, factor);
  else
    hipLaunchKernelGGL((rmsnorm_rows_kernel<16, 1>), dim3(grid), dim3(NT), 0, st, (const uint16_t*)x, x_rs, (uint16_t*)out, o_rs, weight, rows,
                       dim, eps, factor);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

int launch_add_rmsnorm_rows(const void* x, int64_t x_rs, const void* delta, int64_t d_rs, void* x_out, int64_t xo_rs, void* out,
                            int64_t o_rs, const float* weight, int64_t rows, int dim, float eps, hipStream_t st) {
  if (rows == 0) return KVX_OK;
  const float factor = 1.0f / sqrtf((float)dim);
  const unsigned grid = (unsigned)((rows + NT / 64 - 1) / (NT / 64));
  if (workgroup_per_row(rows, dim))
    hipLaunchKernelGGL((add_rmsnorm_rows_kernel<4, NT / 64>), dim3((unsigned)rows), dim3(NT), 0, st, (const uint16_t*)x, x_rs,
                       (const uint16_t*)delta, d_rs, (uint16_t*)x_out, xo_rs, (uint16_t*)out, o_rs, weight, rows, dim, eps, factor);
  else if ((dim / 8 + 63) / 64 <= 4)
    hipLaunchKernelGGL((add_rmsnorm_rows_kernel<4, 1>), dim3(grid), dim3(NT), 0, st, (const uint16_t*)x, x_rs, (const uint16_t*)delta, d_rs,
                       (uint16_t*)x_out, xo_rs, (uint16_t*)out, o_rs, weight, rows, dim, eps, factor);
  else
    hipLaunchKernelGGL((add_rmsnorm_rows_kernel<16, 1>), dim3(grid), dim3(NT), 0, st, (const uint16_t*)x, x_rs, (const uint16_t*)delta, d_rs,
                       (uint16_t*)x_out, xo_rs, (uint16_t*)out, o_rs, weight, rows, dim, eps, factor);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

int launch_swiglu_rows(const void* gate_up, int64_t g_rs, void* out, int64_t o_rs, int64_t rows, int dim, hipStream_t st) {
  const int64_t total = rows * (dim / 8);
  if (total == 0) return KVX_OK;
  hipLaunchKernelGGL(swiglu_rows_kernel, dim3((unsigned)((total + NT - 1) / NT)), dim3(NT), 0, st, (const uint16_t*)gate_up, g_rs,
                     (uint16_t*)out, o_rs, rows, dim);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

int launch_qk_norm_rope(void* qkv, int64_t sb, int64_t stt, int B, int num, int Hq, int Hkv, int D, const float* qw, const float* kw,
                        float eps, const float* cos_t, const float* sin_t, int input_pos, hipStream_t st) {
  const int64_t total = (int64_t)B * num * (Hq + Hkv);
  if (total == 0) return KVX_OK;
  const float factor = 1.0f / sqrtf((float)D);
  const int rpb = NT / (D / 8);
  const unsigned grid = (unsigned)((total + rpb - 1) / rpb);
  if (D == 256)
    hipLaunchKernelGGL(qk_norm_rope_kernel<256>, dim3(grid), dim3(NT), 0, st, (uint16_t*)qkv, sb, stt, B, num, Hq, Hkv, qw, kw, eps, factor,
                       cos_t, sin_t, input_pos);
  else if (D == 128)
    hipLaunchKernelGGL(qk_norm_rope_kernel<128>, dim3(grid), dim3(NT), 0, st, (uint16_t*)qkv, sb, stt, B, num, Hq, Hkv, qw, kw, eps, factor,
                       cos_t, sin_t, input_pos);
  else
    hipLaunchKernelGGL(qk_norm_rope_kernel<64>, dim3(grid), dim3(NT), 0, st, (uint16_t*)qkv, sb, stt, B, num, Hq, Hkv, qw, kw, eps, factor,
                       cos_t, sin_t, input_pos);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

}  // namespace kvx
