// Per-key score-sums W[b,h,k] = (1/G) sum_{i,g} exp2(c * q_{i,g}.k - lse2[b,i,h*G+g]) over the visible
// (query, key) pairs, for gfx950.
//
// Reference behaviour: keys_values/attention/flashinfer_wrapper.py:51-150 (_score_sum_kernel) and
// :156-273 (host side, division by the group size); the value it must equal is
// keys_values/attention/base.py:707-725 (mean over the group, sum over queries).
//
// Key-stationary: a wavefront keeps the K rows of its 64 keys in registers as MFMA B operands for
// the whole kernel and owns those 64 outputs, so W needs no atomics and is bit-reproducible. The
// G*q_len packed query rows (row r = query r / G, head r % G) stream through LDS in tiles of 64 rows,
// double-buffered, shared by the four or eight wavefronts of the workgroup (256 or 512 keys per workgroup).
// S = Q K^T is computed with rows along M, so a lane owns one key column: the sum over queries is a
// per-lane running sum and the two halves of the wavefront are added once at the end.
#include <type_traits>

#include "kvx_common.h"

namespace kvx {
namespace {

constexpr int BQ = 64;    // query rows per LDS tile
constexpr int NW = 64;    // keys per wavefront
// Wavefronts per workgroup, a template argument W: 8 (512 keys per workgroup, one workgroup per compute unit: the
// Q tile staged into LDS serves twice the keys, 4 % on the kernel) when that still gives every compute unit a
// workgroup, else 4 (256 keys, two workgroups per compute unit).

struct ScoreParams {
  const uint16_t* q;
  const void* k;
  const float* k_scale;
  const int32_t* k_zp;
  const int32_t* tp;
  const float* lse;
  float* w;
  float* part;           // query rows split over several workgroups: (splits, B, Hkv, kv_len) partial sums, else NULL
  int32_t tiles_per_z;   // query tiles per split
  int32_t B, Hq, Hkv, G, q_len, kv_len, R, input_pos;
  float c, inv_g;
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, qs_sb, qs_sh, tp_sb, tp_sh;
};

template <int D>
struct alignas(16) Smem {
  static constexpr int QCH16 = D / 8 + 1;  // 16-byte chunks per row incl. pad (conflict-free ds_read_b128)
  u32x4_t q[2][BQ][QCH16];
  float lse[3][BQ];   // read one phase later than q, hence one more buffer
  int32_t qpos[3][BQ];
};

template <int D, int W>
struct QStage {
  static constexpr int QCH = (BQ * D / 8) / (64 * W);  // W = 4: 4 (D=128), 2 (D=64)
  u32x4_t qr[QCH];
  float lse;
  int32_t qpos;
};

// Streams the packed query rows (row r = query r / G, head r % G) of one (batch, KV head) pair.
// The (query, head) of each row this thread loads is advanced incrementally from tile to tile,
// so the loop has no integer division.
template <int D, int W>
struct QLoader {
  static constexpr int NTHREADS = 64 * W;
  static constexpr int CPR = D / 8;
  static constexpr int RPI = NTHREADS / CPR;
  static constexpr int QCH = QStage<D, W>::QCH;
  const uint16_t* qbase;  // (b, first head of the group)
  const float* lbase;     // lse + b * q_len * Hq + kvh * G
  int64_t q_sh, q_st;
  int G, R, Hq, input_pos, row_in, col;
  int qi[QCH], g[QCH];    // row of chunk i in the current tile
  int lqi, lg;            // row of the lse / position this thread stages (tid < BQ)
  int dq, dg;             // BQ / G, BQ % G
  const uint16_t* src[QCH];  // dg == 0: address of chunk i in the current tile
  int64_t step;              // dg == 0: elements between consecutive tiles

  __device__ __forceinline__ void init(const ScoreParams& p, int b, int kvh, int tid, int row_start) {
    col = tid % CPR;
    row_in = tid / CPR;
    G = p.G; R = p.R; Hq = p.Hq; input_pos = p.input_pos;
    q_sh = p.q_sh; q_st = p.q_st;
    qbase = p.q + b * p.q_sb + (int64_t)(kvh * p.G) * p.q_sh;
    lbase = p.lse + (int64_t)b * p.q_len * p.Hq + kvh * p.G;
    dq = BQ / G; dg = BQ % G;
#pragma unroll
    for (int i = 0; i < QCH; ++i) {
      const int r = row_start + row_in + i * RPI;
      qi[i] = r / G;
      g[i] = r % G;
      src[i] = qbase + (int64_t)g[i] * q_sh + (int64_t)qi[i] * q_st + col * 8;
    }
    step = (int64_t)dq * q_st;
    lqi = (row_start + tid) / G;
    lg = (row_start + tid) % G;
  }

  // fetch the tile whose first row is row0, then step the row bookkeeping to the next tile
  __device__ __forceinline__ void fetch(QStage<D, W>& s, int row0, int tid) {
    if (dg == 0) {
      // G divides the tile height: every row keeps its head and moves by BQ / G queries per tile.
      // Rows past the end read row 0 (finite data); their lse = +inf makes their weight zero.
#pragma unroll
      for (int i = 0; i < QCH; ++i) {
        const bool ok = row0 + row_in + i * RPI < R;
        s.qr[i] = *(const u32x4_t*)(ok ? src[i] : qbase);
        src[i] += step;
      }
    } else {
#pragma unroll
      for (int i = 0; i < QCH; ++i) {
        const bool ok = row0 + row_in + i * RPI < R;
        const uint16_t* ptr = qbase + (int64_t)g[i] * q_sh + (int64_t)(ok ? qi[i] : 0) * q_st + col * 8;
        s.qr[i] = *(const u32x4_t*)(ok ? ptr : qbase);
        qi[i] += dq;
        g[i] += dg;
        if (g[i] >= G) {
          g[i] -= G;
          qi[i] += 1;
        }
      }
    }
    if (tid < BQ) {
      const bool ok = row0 + tid < R;
      // rows past the end get lse = +inf so that exp2(... - lse) = 0
      s.lse = ok ? lbase[(int64_t)lqi * Hq + lg] : INFINITY;
      s.qpos = ok ? input_pos + lqi : INT_MAX;
      lqi += dq;
      lg += dg;
      if (lg >= G) {
        lg -= G;
        lqi += 1;
      }
    }
  }

  __device__ __forceinline__ void commit(const QStage<D, W>& s, Smem<D>& sm, int buf, int buf3, int tid) const {
#pragma unroll
    for (int i = 0; i < QCH; ++i) sm.q[buf][row_in + i * RPI][col] = s.qr[i];
    if (tid < BQ) {
      sm.lse[buf3][tid] = s.lse;
      sm.qpos[buf3][tid] = s.qpos;
    }
  }
};

// QSPLIT: the query rows are split over blockIdx.z (short caches that would otherwise leave compute units
// idle); every split writes its sums to p.part and a second kernel adds them in a fixed order.
template <int D, int KV, int W, bool QSPLIT>
__global__ __launch_bounds__(64 * W, D <= 128 ? 2 : 1) void score_sum_kernel(const ScoreParams p) {
  constexpr int BK = NW * W;  // keys per workgroup
  constexpr bool F16 = KV == KVX_KV_F16;  // element type of q and k
  __shared__ Smem<D> sm;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 31;
  const int h = lane >> 5;
  const int group = blockIdx.x;  // fastest: (b, kvh), keeps one KV head's Q stream on one XCD
  const int b = group / p.Hkv, kvh = group % p.Hkv;
  const int key0 = blockIdx.y * BK + wave * NW;

  // K fragments (B operand): lane holds key column n of tile nt, d = 16 j + 8 h .. +8
  u32x4_t kf[2][D / 16];
  int32_t tpk[2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const int key = key0 + nt * 32 + n;
    const bool ok = key < p.kv_len;
    tpk[nt] = ok ? (p.tp ? p.tp[b * p.tp_sb + kvh * p.tp_sh + key] : key) : INT_MAX;
    if constexpr (kv_is_plain(KV)) {
      const uint16_t* kp = (const uint16_t*)p.k + b * p.k_sb + kvh * p.k_sh + (int64_t)key * p.k_st;
#pragma unroll
      for (int j = 0; j < D / 16; ++j) {
        u32x4_t t = ok ? *(const u32x4_t*)(kp + 16 * j + 8 * h) : u32x4_t{0, 0, 0, 0};
        kf[nt][j] = t;
      }
    } else {
      const uint8_t* kp = (const uint8_t*)p.k + b * p.k_sb + kvh * p.k_sh + (int64_t)key * p.k_st;
      const int64_t so = b * p.qs_sb + kvh * p.qs_sh + key;
      const float sc = ok ? p.k_scale[so] : 0.0f;
      const int32_t zp = ok ? p.k_zp[so] : 0;
#pragma unroll
      for (int j = 0; j < D / 16; ++j) {
        u32x2_t cc;
        if constexpr (KV == KVX_KV_U4) {  // chunk 2j + h of the row: one nibble of 8 bytes
          cc = ok ? *(const u32x2_t*)(kp + u4_byte_off<D>(2 * j + h)) : u32x2_t{0, 0};
          cc = u4_codes(cc, u4_shift<D>(2 * j + h));
        } else {
          cc = ok ? *(const u32x2_t*)(kp + 16 * j + 8 * h) : u32x2_t{0, 0};
        }
        kf[nt][j] = dequant_words(cc[0], cc[1], zp, sc);
      }
    }
  }
  // Largest position among this wavefront's keys: query tiles whose smallest position is at least
  // that need no mask at all (true for every key written before the current chunk).
  int tpmax = max(tpk[0], tpk[1]);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) tpmax = max(tpmax, __shfl_xor(tpmax, off, 64));
  tpmax = __builtin_amdgcn_readfirstlane(tpmax);

  float wacc[2] = {0.0f, 0.0f};
  const int tbase = QSPLIT ? (int)blockIdx.z * p.tiles_per_z : 0;  // first query tile of this workgroup
  const int num_qt = QSPLIT ? min(p.tiles_per_z, (p.R + BQ - 1) / BQ - tbase) : (p.R + BQ - 1) / BQ;
  QLoader<D, W> ld;
  ld.init(p, b, kvh, tid, tbase * BQ);
  QStage<D, W> st;

  // S block = 32 query rows x 64 keys: Q rows come from LDS (A operand), K sits in registers.
  auto mfma_block = [&](f32x16_t (&s)[2], int buf, int mt) {
#pragma unroll
    for (int j = 0; j < D / 16; ++j) {
      const u32x4_t qq = sm.q[buf][mt * 32 + n][2 * j + h];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        if (j == 0) {
          const f32x16_t zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          s[nt] = mfma_32x32x16<F16>(qq, kf[nt][j], zero);
        } else {
          s[nt] = mfma_32x32x16<F16>(qq, kf[nt][j], s[nt]);
        }
      }
    }
  };
  // p = exp2(c S - lse) summed over the block's rows; accumulator rows are 8 a + 4 h + (0..3)
  auto valu_block = [&](auto mask_tag, const f32x16_t (&s)[2], int buf3, int mt) {
    constexpr bool MASK = decltype(mask_tag)::value;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const f32x4_t ls = *(const f32x4_t*)&sm.lse[buf3][mt * 32 + 8 * a + 4 * h];
      int4 qp = {0, 0, 0, 0};
      if constexpr (MASK) qp = *(const int4*)&sm.qpos[buf3][mt * 32 + 8 * a + 4 * h];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        float e0 = fast_exp2(fmaf(s[nt][4 * a + 0], p.c, -ls[0]));
        float e1 = fast_exp2(fmaf(s[nt][4 * a + 1], p.c, -ls[1]));
        float e2 = fast_exp2(fmaf(s[nt][4 * a + 2], p.c, -ls[2]));
        float e3 = fast_exp2(fmaf(s[nt][4 * a + 3], p.c, -ls[3]));
        if constexpr (MASK) {
          e0 = tpk[nt] > qp.x ? 0.0f : e0;
          e1 = tpk[nt] > qp.y ? 0.0f : e1;
          e2 = tpk[nt] > qp.z ? 0.0f : e2;
          e3 = tpk[nt] > qp.w ? 0.0f : e3;
        }
        wacc[nt] += (e0 + e1) + (e2 + e3);
      }
    }
  };
  // one matrix instruction, its share of the LDS reads, then its share of the other block's
  // vector work (6 or 10 instructions per matrix instruction, 2 of them transcendental)
  auto interleave = [&](auto mask_tag) {
    constexpr bool MASK = decltype(mask_tag)::value;
    // the first LDS reads go out ahead of the first matrix instruction, so that every operand has
    // been on its way for several steps when its (in-order) consumer is reached
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
    for (int i = 0; i < 2 * (D / 16); ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, MASK ? 8 * 16 / (2 * (D / 16)) : 4 * 16 / (2 * (D / 16)), 0);
      __builtin_amdgcn_sched_group_barrier(0x400, 2 * 16 / (2 * (D / 16)), 0);
    }
  };

  ld.fetch(st, tbase * BQ, tid);
  ld.commit(st, sm, 0, 0, tid);
  if (num_qt > 1) ld.fetch(st, (tbase + 1) * BQ, tid);
  __syncthreads();
  f32x16_t sa[2], sb[2];  // blocks 0 and 1 of the current tile
  mfma_block(sa, 0, 0);

  // Software pipeline: the matrix work of one block runs under the vector work of the block before.
  // Tile t + 1 is committed at the start of iteration t and first read after the barrier inside it.
  for (int t = 0; t < num_qt; ++t) {
    const int buf = t & 1, buf3 = t % 3;
    const bool more = t + 1 < num_qt;
    if (more) {
      ld.commit(st, sm, buf ^ 1, (t + 1) % 3, tid);
      if (t + 2 < num_qt) ld.fetch(st, (tbase + t + 2) * BQ, tid);
    }
    // issue priority: lowest in the first half of a tile, highest on the way to the barrier, so that the
    // four wavefronts of a workgroup wait less for each other (about 1 % on the kernel)
    __builtin_amdgcn_s_setprio(0);
    const bool need_mask = tpmax > p.input_pos + ((tbase + t) * BQ) / p.G;
    if (need_mask) {
      mfma_block(sb, buf, 1);
      valu_block(std::true_type{}, sa, buf3, 0);
      interleave(std::true_type{});
    } else {
      mfma_block(sb, buf, 1);
      valu_block(std::false_type{}, sa, buf3, 0);
      interleave(std::false_type{});
    }
    __builtin_amdgcn_s_setprio(3);
    __syncthreads();
    __builtin_amdgcn_s_setprio(1);
    if (more) {
      if (need_mask) {
        mfma_block(sa, buf ^ 1, 0);
        valu_block(std::true_type{}, sb, buf3, 1);
        interleave(std::true_type{});
      } else {
        mfma_block(sa, buf ^ 1, 0);
        valu_block(std::false_type{}, sb, buf3, 1);
        interleave(std::false_type{});
      }
    } else {
      if (need_mask) valu_block(std::true_type{}, sb, buf3, 1);
      else valu_block(std::false_type{}, sb, buf3, 1);
    }
  }

#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const float tot = sum_halves(wacc[nt]);
    const int key = key0 + nt * 32 + n;
    if (h == 0 && key < p.kv_len) {
      if constexpr (QSPLIT) p.part[(((int64_t)blockIdx.z * p.B + b) * p.Hkv + kvh) * p.kv_len + key] = tot;
      else p.w[((int64_t)b * p.Hkv + kvh) * p.kv_len + key] = tot * p.inv_g;
    }
  }
}

// W = (1/G) * (part[0] + part[1] + ...), in that order.
__global__ void score_sum_reduce_kernel(const float* part, float* w, int64_t n, int splits, float inv_g) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float acc = part[i];
  for (int z = 1; z < splits; ++z) acc += part[(int64_t)z * n + i];
  w[i] = acc * inv_g;
}

// Splits of the query rows: none when the keys alone give every compute unit two workgroups of 256 keys; else as
// many as that takes, each at least 8 tiles of 64 rows (the second launch costs a short chunk more than it
// gains), at most 16.
struct ScorePlan {
  int splits, tiles_per_z;
};
ScorePlan score_plan(const kvx_sdpa_args& a) {
  const int G = a.Hq / a.Hkv;
  const int num_qt = (int)(((int64_t)a.q_len * G + BQ - 1) / BQ);
  const int64_t wgs = (int64_t)a.B * a.Hkv * ((a.kv_len + 4 * NW - 1) / (4 * NW));
  int64_t splits = (2 * num_cus() + wgs - 1) / wgs;
  if (splits > num_qt / 8) splits = num_qt / 8;
  if (splits > 16) splits = 16;
  if (splits < 1) splits = 1;
  ScorePlan pl;
  pl.tiles_per_z = (num_qt + (int)splits - 1) / (int)splits;
  pl.splits = (num_qt + pl.tiles_per_z - 1) / pl.tiles_per_z;
  return pl;
}

template <int D, int KV>
int launch_t(const ScoreParams& p, int splits, hipStream_t st) {
  const int groups = p.B * p.Hkv;
  if (splits > 1) {
    hipLaunchKernelGGL((score_sum_kernel<D, KV, 4, true>), dim3(groups, (p.kv_len + 4 * NW - 1) / (4 * NW), splits), dim3(256), 0, st, p);
    KVX_HIP(hipGetLastError());
    const int64_t n = (int64_t)groups * p.kv_len;
    hipLaunchKernelGGL(score_sum_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p.part, p.w, n, splits, p.inv_g);
    KVX_HIP(hipGetLastError());
    return KVX_OK;
  }
  if constexpr (D <= 128) {
    const int wide = (p.kv_len + 8 * NW - 1) / (8 * NW);
    if ((int64_t)groups * wide >= num_cus()) {
      hipLaunchKernelGGL((score_sum_kernel<D, KV, 8, false>), dim3(groups, wide), dim3(512), 0, st, p);
      KVX_HIP(hipGetLastError());
      return KVX_OK;
    }
  }
  hipLaunchKernelGGL((score_sum_kernel<D, KV, 4, false>), dim3(groups, (p.kv_len + 4 * NW - 1) / (4 * NW)), dim3(256), 0, st, p);
  KVX_HIP(hipGetLastError());
  return KVX_OK;
}

}  // namespace

size_t score_sum_workspace(const kvx_sdpa_args& a) {
  const ScorePlan pl = score_plan(a);
  return pl.splits > 1 ? (size_t)pl.splits * a.B * a.Hkv * a.kv_len * sizeof(float) : 0;
}

int launch_score_sum(const kvx_sdpa_args& a, hipStream_t st) {
  // the query rows are split only if the caller's workspace holds the partial sums
  ScorePlan pl = score_plan(a);
  if (pl.splits > 1 && !(a.workspace && a.workspace_bytes >= score_sum_workspace(a) && ((uintptr_t)a.workspace & 15) == 0)) pl.splits = 1;
  ScoreParams p;
  p.part = pl.splits > 1 ? (float*)a.workspace : nullptr;
  p.tiles_per_z = pl.tiles_per_z;
  p.q = (const uint16_t*)a.q;
  p.k = a.k;
  p.k_scale = a.k_scale;
  p.k_zp = a.k_zp;
  p.tp = a.token_positions;
  p.lse = a.lse;
  p.w = a.w;
  p.B = a.B; p.Hq = a.Hq; p.Hkv = a.Hkv; p.G = a.Hq / a.Hkv;
  p.q_len = a.q_len; p.kv_len = a.kv_len; p.R = a.q_len * p.G; p.input_pos = a.input_pos;
  p.c = a.sm_scale * kLog2e;
  p.inv_g = 1.0f / (float)p.G;
  p.q_sb = a.q_stride_b; p.q_sh = a.q_stride_h; p.q_st = a.q_stride_t;
  p.k_sb = a.k_stride_b; p.k_sh = a.k_stride_h; p.k_st = a.k_stride_t;
  p.qs_sb = a.qs_stride_b; p.qs_sh = a.qs_stride_h;
  p.tp_sb = a.tp_stride_b; p.tp_sh = a.tp_stride_h;
  if (a.D == 128) {
    if (a.kv_dtype == KVX_KV_U4) return launch_t<128, KVX_KV_U4>(p, pl.splits, st);
    if (a.kv_dtype == KVX_KV_F16) return launch_t<128, KVX_KV_F16>(p, pl.splits, st);
    return a.kv_dtype == KVX_KV_U8 ? launch_t<128, KVX_KV_U8>(p, pl.splits, st) : launch_t<128, KVX_KV_BF16>(p, pl.splits, st);
  }
  if (a.D == 64) {
    if (a.kv_dtype == KVX_KV_U4) return launch_t<64, KVX_KV_U4>(p, pl.splits, st);
    if (a.kv_dtype == KVX_KV_F16) return launch_t<64, KVX_KV_F16>(p, pl.splits, st);
    return a.kv_dtype == KVX_KV_U8 ? launch_t<64, KVX_KV_U8>(p, pl.splits, st) : launch_t<64, KVX_KV_BF16>(p, pl.splits, st);
  }
  if (a.D == 256 && kv_is_plain(a.kv_dtype))
    return a.kv_dtype == KVX_KV_F16 ? launch_t<256, KVX_KV_F16>(p, pl.splits, st) : launch_t<256, KVX_KV_BF16>(p, pl.splits, st);
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_score_sum: head size %d not in {64, 128, 256} (quantised stores: {64, 128})", a.D);
}

}  // namespace kvx
