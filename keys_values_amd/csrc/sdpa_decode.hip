// Single-token decode attention with per-key score-sums for gfx950 (HBM-bound).
//
// Reference behaviour: keys_values/attention/flashinfer_ops.py:193-275 (sdpa_decode: no mask, the
// weights divided by the group size), keys_values/csrc/kernels/sdpa_decode.cu:616-898 (the kernel
// it calls, which reads K and V once per QUERY head and keeps fp32 logits to turn them into
// weights afterwards, :838-854).
//
// Here one workgroup serves all G query heads of a (batch, KV head, split), so K and V cross HBM
// once. Per block of keys (8192 / G of them) it runs three phases:
//   1. logits = c * K q for the G heads with 16x16x32 bf16 MFMA: a K row is the A operand straight
//      from global memory (16-byte loads, no LDS staging), the G query vectors sit in the B operand.
//      The logits (log2 units) go to LDS and, when weights are wanted, to the fp32 logits scratch.
//   2. with the block maximum known, p = exp2(logit - max) is written back to LDS as bf16 pairs of
//      the two keys a lane will multiply together, and summed in fp32.
//   3. O += p V with v_dot2_f32_bf16 on (key A, key B) pairs: a lane owns 8 consecutive d of the
//      rows it loads (16-byte loads, a wavefront covers whole contiguous rows), accumulates in fp32
//      registers and the partial sums are reduced across lanes and wavefronts once at the end.
// A merge kernel combines the splits and produces the base-2 log-sum-exp; a last streaming kernel
// turns the stored logits into W = (1/G) sum_g exp2(logit_g - lse_g). No float atomics anywhere.
#include "kvx_common.h"

namespace kvx {
namespace {

constexpr int NTHREADS = 256;
constexpr int WAVES = 4;

struct DecodeParams {
  const uint16_t* q;
  const void* k;
  const void* v;
  const float* k_scale;
  const int32_t* k_zp;
  const float* v_scale;
  const int32_t* v_zp;
  uint16_t* o;
  float* lse_out;  // user (B, 1, Hq) or NULL
  float* w;        // user (B, Hkv, kv_len) or NULL
  float* logits;   // (B, Hq, Tpad)
  float* part_o;   // (B, Hq, S, D)
  float* part_ml;  // (B, Hq, S, 2)
  float* lse_ws;   // (B, Hq)
  int32_t B, Hq, Hkv, kv_len, Tpad, num_splits, keys_per_split;
  float c;
  int64_t q_sb, q_sh, k_sb, k_sh, k_st, v_sb, v_sh, v_st, o_sb, o_sh, qs_sb, qs_sh;
};

__device__ __forceinline__ u32x4_t dq8(uint32_t c0, uint32_t c1, int32_t zp, float scale) {
  u32x4_t r;
  r[0] = dequant_pair(c0 & 0xff, (c0 >> 8) & 0xff, zp, scale);
  r[1] = dequant_pair((c0 >> 16) & 0xff, c0 >> 24, zp, scale);
  r[2] = dequant_pair(c1 & 0xff, (c1 >> 8) & 0xff, zp, scale);
  r[3] = dequant_pair((c1 >> 16) & 0xff, c1 >> 24, zp, scale);
  return r;
}

template <int D, int G, bool U8>
__global__ __launch_bounds__(NTHREADS) void decode_split_kernel(const DecodeParams p) {
  constexpr int KPB = 8192 / G;   // keys per block held in LDS
  constexpr int LPR = D / 8;      // lanes per V row
  constexpr int KPI = 64 / LPR;   // V rows per load instruction of a wavefront
  constexpr int KS = D / 32;      // MFMA k-steps per key group
  __shared__ float lg[KPB * G];          // logits [key][head], log2 units
  __shared__ uint32_t pp[(KPB / 2) * G]; // bf16 pairs (p[key A], p[key B]) [pair][head]
  __shared__ float smx[WAVES][G];        // per-wavefront maxima, later per-wavefront sums

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int k_begin = split * p.keys_per_split;
  const int k_end = min(k_begin + p.keys_per_split, p.kv_len);

  // B operand: column nn = query head (zero beyond G), d = 32 j + 8 hq .. +8
  const int nn = lane & 15, hq = lane >> 4;
  bf16x8_t qf[KS];
#pragma unroll
  for (int j = 0; j < KS; ++j) {
    u32x4_t t = {0, 0, 0, 0};
    if (nn < G) t = *(const u32x4_t*)(p.q + b * p.q_sb + (int64_t)(kvh * G + nn) * p.q_sh + 32 * j + 8 * hq);
    qf[j] = as_bf16x8(t);
  }

  const uint8_t* kbase = (const uint8_t*)p.k + (b * p.k_sb + kvh * p.k_sh) * (U8 ? 1 : 2);
  const uint8_t* vbase = (const uint8_t*)p.v + (b * p.v_sb + kvh * p.v_sh) * (U8 ? 1 : 2);
  const int64_t qs_off = b * p.qs_sb + kvh * p.qs_sh;

  float acc[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.0f;
  float m_run[G], l_run[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m_run[g] = -INFINITY;
    l_run[g] = 0.0f;
  }

  for (int blk0 = k_begin; blk0 < k_end; blk0 += KPB) {
    const int nk = min(KPB, k_end - blk0);
    const int ngroups = (nk + 15) / 16;
    // ---- phase 1: logits ----------------------------------------------------------------
    float mloc = -INFINITY;  // lanes with nn < G: max over their keys for head nn
    for (int gi = wave; gi < ngroups; gi += WAVES) {
      const int key = blk0 + gi * 16 + nn;  // A operand row of this lane
      const bool ok = key < k_end;
      f32x4_t s = {0, 0, 0, 0};
      if constexpr (!U8) {
        const uint16_t* kp = (const uint16_t*)kbase + (int64_t)key * p.k_st + 8 * hq;
        u32x4_t kr[KS];
#pragma unroll
        for (int j = 0; j < KS; ++j) kr[j] = ok ? *(const u32x4_t*)(kp + 32 * j) : u32x4_t{0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < KS; ++j) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kr[j]), qf[j], s, 0, 0, 0);
      } else {
        const uint8_t* kp = kbase + (int64_t)key * p.k_st + 8 * hq;
        u32x2_t kr[KS];
#pragma unroll
        for (int j = 0; j < KS; ++j) kr[j] = ok ? *(const u32x2_t*)(kp + 32 * j) : u32x2_t{0, 0};
        const float sc = ok ? p.k_scale[qs_off + key] : 0.0f;
        const int32_t zp = ok ? p.k_zp[qs_off + key] : 0;
#pragma unroll
        for (int j = 0; j < KS; ++j)
          s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(dq8(kr[j][0], kr[j][1], zp, sc)), qf[j], s, 0, 0, 0);
      }
      // accumulator: column nn = head, rows 4 hq + i = keys of the group
      if (nn < G) {
        const int kl = gi * 16 + 4 * hq;  // local key of row i = 0
        f32x4_t t;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          t[i] = (blk0 + kl + i < k_end) ? s[i] * p.c : -INFINITY;
          mloc = fmaxf(mloc, t[i]);
          lg[(kl + i) * G + nn] = t[i];
        }
        if (p.logits) *(f32x4_t*)(p.logits + ((int64_t)b * p.Hq + kvh * G + nn) * p.Tpad + blk0 + kl) = t;
      }
    }
    // keys of the last, partial pair group that phase 1 did not touch
    for (int i = ngroups * 16 * G + tid; i < ((nk + 2 * KPI - 1) / (2 * KPI)) * (2 * KPI) * G; i += NTHREADS) lg[i] = -INFINITY;
    // block maximum per head
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    if (lane < G) smx[wave][lane] = mloc;
    __syncthreads();
    float m_new[G], alpha[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mb = smx[0][g];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) mb = fmaxf(mb, smx[w][g]);
      m_new[g] = fmaxf(m_run[g], mb);  // finite: every block holds at least one key
      alpha[g] = fast_exp2(m_run[g] - m_new[g]);
    }
    // ---- phase 2: p = exp2(logit - max) as bf16 pairs (key, key + KPI) ---------------------
    const int npairs = ((nk + 2 * KPI - 1) / (2 * KPI)) * KPI;
    float lsum[G];
#pragma unroll
    for (int g = 0; g < G; ++g) lsum[g] = 0.0f;
    for (int pi = tid; pi < npairs; pi += NTHREADS) {
      const int ka = (pi / KPI) * (2 * KPI) + (pi % KPI);
      const int kb = ka + KPI;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const float pa = fast_exp2(lg[ka * G + g] - m_new[g]);
        const float pb = fast_exp2(lg[kb * G + g] - m_new[g]);
        lsum[g] += pa + pb;
        pp[pi * G + g] = pack_bf16(pa, pb);
      }
    }
    __syncthreads();  // smx consumed, pp complete
    // ---- phase 3: O += p V ------------------------------------------------------------------
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] *= alpha[g];
    const int kk = lane / LPR, dc = lane % LPR;
    const int niter = npairs / KPI;  // each iteration of a wavefront covers 2 KPI keys
    for (int it = wave; it < niter; it += WAVES) {
      const int ka = blk0 + it * 2 * KPI + kk;
      const int kb = ka + KPI;
      u32x4_t va, vb;
      if constexpr (!U8) {
        va = ka < k_end ? *(const u32x4_t*)((const uint16_t*)vbase + (int64_t)ka * p.v_st + 8 * dc) : u32x4_t{0, 0, 0, 0};
        vb = kb < k_end ? *(const u32x4_t*)((const uint16_t*)vbase + (int64_t)kb * p.v_st + 8 * dc) : u32x4_t{0, 0, 0, 0};
      } else {
        const u32x2_t ca = ka < k_end ? *(const u32x2_t*)(vbase + (int64_t)ka * p.v_st + 8 * dc) : u32x2_t{0, 0};
        const u32x2_t cb = kb < k_end ? *(const u32x2_t*)(vbase + (int64_t)kb * p.v_st + 8 * dc) : u32x2_t{0, 0};
        va = dq8(ca[0], ca[1], ka < k_end ? p.v_zp[qs_off + ka] : 0, ka < k_end ? p.v_scale[qs_off + ka] : 0.0f);
        vb = dq8(cb[0], cb[1], kb < k_end ? p.v_zp[qs_off + kb] : 0, kb < k_end ? p.v_scale[qs_off + kb] : 0.0f);
      }
      uint32_t pr[G];
#pragma unroll
      for (int g = 0; g < G; ++g) pr[g] = pp[(it * KPI + kk) * G + g];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bf16x2_t lo = __builtin_bit_cast(bf16x2_t, __builtin_amdgcn_perm(vb[e], va[e], 0x05040100u));
        const bf16x2_t hi = __builtin_bit_cast(bf16x2_t, __builtin_amdgcn_perm(vb[e], va[e], 0x07060302u));
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const bf16x2_t pg = __builtin_bit_cast(bf16x2_t, pr[g]);
          acc[g][2 * e] = __builtin_amdgcn_fdot2_f32_bf16(lo, pg, acc[g][2 * e], false);
          acc[g][2 * e + 1] = __builtin_amdgcn_fdot2_f32_bf16(hi, pg, acc[g][2 * e + 1], false);
        }
      }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      l_run[g] = l_run[g] * alpha[g] + lsum[g];  // per-thread share of the sum
      m_run[g] = m_new[g];
    }
    __syncthreads();  // lg / pp are rewritten by the next block
  }

  // ---- reduce the partial O over the lanes that share a d chunk, then over wavefronts ---------
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = acc[g][e];
#pragma unroll
      for (int off = LPR; off < 64; off <<= 1) x += __shfl_xor(x, off, 64);
      acc[g][e] = x;
    }
    float s = l_run[g];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    l_run[g] = s;
  }
  // lg is free now (the loop ended with a barrier): reuse it as red[wave][head][d]
  float* red = lg;
  if (lane < LPR) {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) red[(wave * G + g) * D + lane * 8 + e] = acc[g][e];
  }
  if (lane == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) smx[wave][g] = l_run[g];
  }
  __syncthreads();
  for (int i = tid; i < G * D; i += NTHREADS) {
    const int g = i / D, d = i % D;
    float x = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) x += red[(w * G + g) * D + d];
    p.part_o[(((int64_t)b * p.Hq + kvh * G + g) * p.num_splits + split) * D + d] = x;
  }
  if (tid == 0) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float s = 0.0f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) s += smx[w][g];
      const int64_t o = (((int64_t)b * p.Hq + kvh * G + g) * p.num_splits + split) * 2;
      p.part_ml[o] = m_run[g];
      p.part_ml[o + 1] = s;
    }
  }
}

// One workgroup of D threads per (b, query head): combine the splits.
template <int D>
__global__ void decode_merge_kernel(const DecodeParams p) {
  const int bh = blockIdx.x;
  const int b = bh / p.Hq, hqi = bh % p.Hq;
  const int d = threadIdx.x;
  const float* ml = p.part_ml + (int64_t)bh * p.num_splits * 2;
  float M = -INFINITY;
  for (int s = 0; s < p.num_splits; ++s) M = fmaxf(M, ml[2 * s]);
  float L = 0.0f, acc = 0.0f;
  for (int s = 0; s < p.num_splits; ++s) {
    const float w = fast_exp2(ml[2 * s] - M);
    L += ml[2 * s + 1] * w;
    acc += p.part_o[((int64_t)bh * p.num_splits + s) * D + d] * w;
  }
  const float r = acc / L;
  const float other = __shfl_xor(r, 1, 64);
  if ((d & 1) == 0) *(uint32_t*)(p.o + b * p.o_sb + hqi * p.o_sh + d) = pack_bf16(r, other);
  if (d == 0) {
    const float lse = M + fast_log2(L);
    p.lse_ws[bh] = lse;
    if (p.lse_out) p.lse_out[bh] = lse;
  }
}

// W[b, kvh, k] = (1/G) sum_g exp2(logit[b, kvh*G+g, k] - lse[b, kvh*G+g]); 4 keys per lane.
template <int G>
__global__ __launch_bounds__(256) void decode_weights_kernel(const DecodeParams p) {
  const int kvh = blockIdx.y, b = blockIdx.z;
  const int k0 = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (k0 >= p.kv_len) return;
  f32x4_t acc = {0, 0, 0, 0};
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int64_t bh = (int64_t)b * p.Hq + kvh * G + g;
    const float lse = p.lse_ws[bh];
    const f32x4_t t = *(const f32x4_t*)(p.logits + bh * p.Tpad + k0);
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] += fast_exp2(t[e] - lse);
  }
  acc *= 1.0f / (float)G;
  float* wr = p.w + ((int64_t)b * p.Hkv + kvh) * p.kv_len;
  if (k0 + 3 < p.kv_len && (p.kv_len & 3) == 0) {
    *(f32x4_t*)(wr + k0) = acc;
  } else {
    for (int e = 0; e < 4 && k0 + e < p.kv_len; ++e) wr[k0 + e] = acc[e];
  }
}

struct Plan {
  int G, kpb, num_splits, keys_per_split, Tpad;
  size_t off_logits, off_part_o, off_part_ml, off_lse, total;
};

Plan make_plan(const kvx_sdpa_args& a) {
  Plan pl;
  pl.G = a.Hq / a.Hkv;
  pl.kpb = 8192 / pl.G;
  int splits = a.num_splits > 0 ? a.num_splits : (a.kv_len + pl.kpb - 1) / pl.kpb;
  splits = max(1, min(splits, 512));
  int kps = (a.kv_len + splits - 1) / splits;
  kps = ((kps + 63) / 64) * 64;  // keeps the 16-byte logits stores aligned
  pl.keys_per_split = kps;
  pl.num_splits = (a.kv_len + kps - 1) / kps;
  pl.Tpad = ((a.kv_len + 63) / 64) * 64;
  size_t off = 0;
  pl.off_logits = off;
  off += a.w ? (size_t)a.B * a.Hq * pl.Tpad * 4 : 0;
  pl.off_part_o = off;
  off += (size_t)a.B * a.Hq * pl.num_splits * a.D * 4;
  pl.off_part_ml = off;
  off += (size_t)a.B * a.Hq * pl.num_splits * 2 * 4;
  pl.off_lse = off;
  off += (size_t)a.B * a.Hq * 4;
  pl.total = (off + 255) & ~(size_t)255;
  return pl;
}

template <int D, int G>
int launch_dg(const DecodeParams& p, bool u8, hipStream_t st) {
  dim3 grid(p.num_splits, p.Hkv, p.B);
  if (u8) hipLaunchKernelGGL((decode_split_kernel<D, G, true>), grid, dim3(NTHREADS), 0, st, p);
  else hipLaunchKernelGGL((decode_split_kernel<D, G, false>), grid, dim3(NTHREADS), 0, st, p);
  KVX_HIP(hipGetLastError());
  hipLaunchKernelGGL((decode_merge_kernel<D>), dim3(p.B * p.Hq), dim3(D), 0, st, p);
  KVX_HIP(hipGetLastError());
  if (p.w) {
    hipLaunchKernelGGL((decode_weights_kernel<G>), dim3((p.kv_len + 1023) / 1024, p.Hkv, p.B), dim3(256), 0, st, p);
    KVX_HIP(hipGetLastError());
  }
  return KVX_OK;
}

template <int D>
int launch_d(const DecodeParams& p, int G, bool u8, hipStream_t st) {
  switch (G) {
    case 1: return launch_dg<D, 1>(p, u8, st);
    case 2: return launch_dg<D, 2>(p, u8, st);
    case 4: return launch_dg<D, 4>(p, u8, st);
    case 8: return launch_dg<D, 8>(p, u8, st);
  }
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_sdpa_decode: group size %d not in {1, 2, 4, 8}", G);
}

}  // namespace

size_t sdpa_decode_workspace(const kvx_sdpa_args& a) { return make_plan(a).total; }

int launch_sdpa_decode(const kvx_sdpa_args& a, hipStream_t st) {
  const Plan pl = make_plan(a);
  KVX_REQUIRE(a.workspace && a.workspace_bytes >= pl.total, KVX_ERR_WORKSPACE,
              "kvx_sdpa_decode: workspace of %zu bytes needed, %zu given", pl.total, a.workspace_bytes);
  DecodeParams p;
  char* ws = (char*)a.workspace;
  p.q = (const uint16_t*)a.q;
  p.k = a.k;
  p.v = a.v;
  p.k_scale = a.k_scale; p.k_zp = a.k_zp; p.v_scale = a.v_scale; p.v_zp = a.v_zp;
  p.o = (uint16_t*)a.o;
  p.lse_out = a.lse;
  p.w = a.w;
  p.logits = a.w ? (float*)(ws + pl.off_logits) : nullptr;
  p.part_o = (float*)(ws + pl.off_part_o);
  p.part_ml = (float*)(ws + pl.off_part_ml);
  p.lse_ws = (float*)(ws + pl.off_lse);
  p.B = a.B; p.Hq = a.Hq; p.Hkv = a.Hkv; p.kv_len = a.kv_len; p.Tpad = pl.Tpad;
  p.num_splits = pl.num_splits; p.keys_per_split = pl.keys_per_split;
  p.c = a.sm_scale * kLog2e;
  p.q_sb = a.q_stride_b; p.q_sh = a.q_stride_h;
  p.k_sb = a.k_stride_b; p.k_sh = a.k_stride_h; p.k_st = a.k_stride_t;
  p.v_sb = a.v_stride_b; p.v_sh = a.v_stride_h; p.v_st = a.v_stride_t;
  p.o_sb = a.o_stride_b; p.o_sh = a.o_stride_h;
  p.qs_sb = a.qs_stride_b; p.qs_sh = a.qs_stride_h;
  const bool u8 = a.kv_dtype == KVX_KV_U8;
  if (a.D == 128) return launch_d<128>(p, pl.G, u8, st);
  if (a.D == 64) return launch_d<64>(p, pl.G, u8, st);
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_sdpa_decode: head size %d not in {64, 128}", a.D);
}

}  // namespace kvx
