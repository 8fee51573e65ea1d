// Chunked-prefill attention for gfx950: O = softmax(s Q K^T + mask) V with the base-2 log-sum-exp.
//
// Reference behaviour: keys_values/attention/base.py:660-742 (eager arithmetic),
// keys_values/csrc/kernels/sdpa_prefill.cu:34-181 (what the FlashInfer prefill returns: O and
// base-2 LSE), keys_values/attention/attention_utils.py:238-247 (mask by token position).
//
// Work decomposition
//   The G query heads that share a KV head are packed into the row dimension: row r of a
//   (batch, KV head) pair is (query r / G, head r % G), R = q_len * G rows in all. A workgroup of
//   four wavefronts owns 128 consecutive rows (32 per wavefront) and walks the key tiles of its KV
//   split, 64 keys at a time, so a K/V tile staged once in LDS serves all G heads.
//   Scores are produced TRANSPOSED, S^T = K Q^T (32x32x16 bf16 MFMA, keys along M, rows along N):
//   every lane then owns one row's statistics (running max and sum) and only the other half of the
//   wavefront holds the remaining keys of that row, so the online softmax needs a single
//   cross-lane exchange per tile. The accumulator layout of S^T is exactly the B-operand layout
//   of the second product O^T = V^T P^T once the 16 keys of a k-step are taken in the order
//   (0..3, 8..11 | 4..7, 12..15); V is therefore staged transposed in LDS with that key order.
//   K/V tiles are double-buffered: the next tile is fetched into registers while the current one
//   is multiplied, and written to the other LDS buffer before the single barrier of the iteration.
#include "kvx_common.h"

namespace kvx {
namespace {

constexpr int BM = 128;  // rows per workgroup
constexpr int BN = 64;   // keys per tile
constexpr int NTHREADS = 256;

struct PrefillParams {
  const uint16_t* q;
  const void* k;
  const void* v;
  const float* k_scale;
  const int32_t* k_zp;
  const float* v_scale;
  const int32_t* v_zp;
  const int32_t* tp;
  uint16_t* o;
  float* lse;
  float* part_o;   // [split][group][R][D] fp32, unnormalised
  float* part_ml;  // [split][group][R][2]  (max in log2 units, sum)
  int32_t B, Hq, Hkv, G, q_len, kv_len, R, input_pos;
  int32_t num_splits, tiles_per_split, num_tiles, m_blocks;
  float c;  // sm_scale * log2(e)
  int64_t q_sb, q_sh, q_st, k_sb, k_sh, k_st, v_sb, v_sh, v_st, o_sb, o_sh, o_st;
  int64_t qs_sb, qs_sh, tp_sb, tp_sh;
};

template <int D>
struct alignas(16) Smem {
  static constexpr int KCH16 = D / 8 + 1;   // 16-byte chunks per K row incl. pad: row stride = 4 banks mod 64,
                                            // so the 16 rows a ds_read_b128 phase touches hit distinct banks
  static constexpr int VCH16 = D / 8 + 4;   // V row stride = 16 banks mod 64: the 4 rows x 64 bytes a pair of
                                            // 16-lane transpose-read groups touches hit distinct banks
  u32x4_t k[2][BN][KCH16];                  // [key][d]
  u32x4_t v[2][BN][VCH16];                  // [key][d]
  int32_t tp[2][BN];
};

typedef short s16x4_t __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i (a = i % 4, r = i / 4) supplies the
// address of 4 consecutive bf16 of "row r, columns 4a..4a+3"; it receives column i of rows 0..3.
__device__ __forceinline__ u32x2_t lds_read_tr16(const void* p) {
  const s16x4_t t = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(p));
  return __builtin_bit_cast(u32x2_t, t);
}

// 8 codes (two dwords) -> 8 bf16 (four dwords)
__device__ __forceinline__ u32x4_t dequant8(uint32_t c0, uint32_t c1, int32_t zp, float scale) {
  u32x4_t r;
  r[0] = dequant_pair(c0 & 0xff, (c0 >> 8) & 0xff, zp, scale);
  r[1] = dequant_pair((c0 >> 16) & 0xff, c0 >> 24, zp, scale);
  r[2] = dequant_pair(c1 & 0xff, (c1 >> 8) & 0xff, zp, scale);
  r[3] = dequant_pair((c1 >> 16) & 0xff, c1 >> 24, zp, scale);
  return r;
}

template <int D, bool U8>
struct Stage {
  // registers holding one prefetched K/V tile of this thread: KCH rows, one 16-byte chunk each
  static constexpr int KCH = (BN * D / 8) / NTHREADS;  // 4 (D=128), 2 (D=64)
  u32x4_t kr[KCH];
  u32x4_t vr[KCH];
  float ks[KCH], vs[KCH];
  int32_t kz[KCH], vz[KCH];
  int32_t tpv;
};

template <int D, bool U8>
struct Loader {
  static constexpr int CPR = D / 8;             // chunks per row
  static constexpr int RPI = NTHREADS / CPR;    // rows per pass of the workgroup
  static constexpr int KCH = Stage<D, U8>::KCH;
  static constexpr int ESZ = U8 ? 1 : 2;        // bytes per element in memory
  const char* kbase;                            // (b, kvh) slice, uniform
  const char* vbase;
  const float* ks;
  const int32_t* kz;
  const float* vs;
  const int32_t* vz;
  const int32_t* tp;                            // may be NULL
  uint32_t koff[KCH], voff[KCH];                // byte offsets of this thread's chunks inside a tile
  int64_t k_tile_bytes, v_tile_bytes;
  int64_t k_st, v_st;
  int row_in, col, kv_len;

  __device__ __forceinline__ void init(const PrefillParams& p, int b, int kvh, int tid) {
    col = tid % CPR;
    row_in = tid / CPR;
    kv_len = p.kv_len;
    k_st = p.k_st;
    v_st = p.v_st;
    kbase = (const char*)p.k + (b * p.k_sb + kvh * p.k_sh) * ESZ;
    vbase = (const char*)p.v + (b * p.v_sb + kvh * p.v_sh) * ESZ;
    const int64_t so = b * p.qs_sb + kvh * p.qs_sh;
    ks = p.k_scale + so;
    kz = p.k_zp + so;
    vs = p.v_scale + so;
    vz = p.v_zp + so;
    tp = p.tp ? p.tp + b * p.tp_sb + kvh * p.tp_sh : nullptr;
    k_tile_bytes = (int64_t)BN * p.k_st * ESZ;
    v_tile_bytes = (int64_t)BN * p.v_st * ESZ;
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      koff[i] = (uint32_t)((row_in + i * RPI) * p.k_st * ESZ + col * 8 * ESZ);
      voff[i] = (uint32_t)((row_in + i * RPI) * p.v_st * ESZ + col * 8 * ESZ);
    }
  }

  __device__ __forceinline__ void fetch(Stage<D, U8>& s, int tile, int tid) const {
    const int key0 = tile * BN;
    const char* kt = kbase + tile * k_tile_bytes;
    const char* vt = vbase + tile * v_tile_bytes;
    if (key0 + BN <= kv_len) {
#pragma unroll
      for (int i = 0; i < KCH; ++i) {
        if constexpr (!U8) {
          s.kr[i] = *(const u32x4_t*)(kt + koff[i]);
          s.vr[i] = *(const u32x4_t*)(vt + voff[i]);
        } else {
          const u32x2_t ck = *(const u32x2_t*)(kt + koff[i]);
          const u32x2_t cv = *(const u32x2_t*)(vt + voff[i]);
          s.kr[i] = u32x4_t{ck[0], ck[1], 0, 0};
          s.vr[i] = u32x4_t{cv[0], cv[1], 0, 0};
          const int key = key0 + row_in + i * RPI;
          s.ks[i] = ks[key];
          s.kz[i] = kz[key];
          s.vs[i] = vs[key];
          s.vz[i] = vz[key];
        }
      }
      if (tid < BN) s.tpv = tp ? tp[key0 + tid] : key0 + tid;
    } else {
      // last, partial tile: rows past the end re-read the last valid row (finite data); their
      // position is INT_MAX, so they are masked for every query and contribute exactly zero
#pragma unroll
      for (int i = 0; i < KCH; ++i) {
        const int key = min(key0 + row_in + i * RPI, kv_len - 1);
        if constexpr (!U8) {
          s.kr[i] = *(const u32x4_t*)(kbase + ((int64_t)key * k_st + col * 8) * ESZ);
          s.vr[i] = *(const u32x4_t*)(vbase + ((int64_t)key * v_st + col * 8) * ESZ);
        } else {
          const u32x2_t ck = *(const u32x2_t*)(kbase + ((int64_t)key * k_st + col * 8));
          const u32x2_t cv = *(const u32x2_t*)(vbase + ((int64_t)key * v_st + col * 8));
          s.kr[i] = u32x4_t{ck[0], ck[1], 0, 0};
          s.vr[i] = u32x4_t{cv[0], cv[1], 0, 0};
          s.ks[i] = ks[key];
          s.kz[i] = kz[key];
          s.vs[i] = vs[key];
          s.vz[i] = vz[key];
        }
      }
      if (tid < BN) {
        const int key = key0 + tid;
        s.tpv = key < kv_len ? (tp ? tp[key] : key) : INT_MAX;
      }
    }
  }

  __device__ __forceinline__ void commit(const Stage<D, U8>& s, Smem<D>& sm, int buf, int tid) const {
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
      u32x4_t kk = s.kr[i], vv = s.vr[i];
      if constexpr (U8) {
        kk = dequant8(kk[0], kk[1], s.kz[i], s.ks[i]);
        vv = dequant8(vv[0], vv[1], s.vz[i], s.vs[i]);
      }
      sm.k[buf][row_in + i * RPI][col] = kk;
      sm.v[buf][row_in + i * RPI][col] = vv;
    }
    if (tid < BN) sm.tp[buf][tid] = s.tpv;
  }
};

template <int D, bool U8>
__global__ __launch_bounds__(NTHREADS, 2) void sdpa_prefill_kernel(const PrefillParams p) {
  __shared__ Smem<D> sm;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n = lane & 31;  // row (query) owned by this lane within the wavefront's 32 rows
  const int h = lane >> 5;  // which half of each 8-wide k group / which 4-row group of the MFMA output

  const int group = blockIdx.x;  // b * Hkv + kvh: fastest-varying so that a KV head stays on one XCD
  const int mblk = blockIdx.y;
  const int split = blockIdx.z;
  const int b = group / p.Hkv;
  const int kvh = group % p.Hkv;

  const int row0w = mblk * BM + wave * 32;
  const int row = row0w + n;
  const bool row_ok = row < p.R;
  const int rowc = row_ok ? row : p.R - 1;
  const int qi = rowc / p.G;
  const int g = rowc % p.G;
  const int qpos = p.input_pos + qi;
  const int qpos_min_w = p.input_pos + min(row0w, p.R - 1) / p.G;

  // Q fragments (B operand): lane holds row n, d = 16 j + 8 h .. +8
  bf16x8_t qf[D / 16];
  {
    const uint16_t* qp = p.q + b * p.q_sb + (int64_t)(kvh * p.G + g) * p.q_sh + (int64_t)qi * p.q_st;
#pragma unroll
    for (int j = 0; j < D / 16; ++j) {
      u32x4_t t = row_ok ? *(const u32x4_t*)(qp + 16 * j + 8 * h) : u32x4_t{0, 0, 0, 0};
      qf[j] = as_bf16x8(t);
    }
  }

  const int tile_begin = split * p.tiles_per_split;
  const int tile_end = min(tile_begin + p.tiles_per_split, p.num_tiles);

  f32x16_t o[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.0f;
  float m = -INFINITY;  // running max of the raw (unscaled) scores of this row
  float l = 0.0f;       // this lane's share of the running sum

  // transpose-read addressing of V: in its group of 16 lanes this lane points at key row (i / 4)
  // and at d columns 4 (i % 4) .. +3 of the 16 d columns the group produces
  const int li = lane & 15;
  const int v_row_off = (li >> 2) + 4 * h;                      // + 32 mt + 16 j (+ 8)
  const int v_col_off = 16 * ((lane >> 4) & 1) + 4 * (li & 3);  // + 32 dt, in bf16 elements

  Loader<D, U8> ld;
  ld.init(p, b, kvh, tid);
  Stage<D, U8> st;
  if (tile_begin < tile_end) {
    ld.fetch(st, tile_begin, tid);
    ld.commit(st, sm, 0, tid);
    if (tile_begin + 1 < tile_end) ld.fetch(st, tile_begin + 1, tid);
  }
  __syncthreads();

  for (int t = tile_begin; t < tile_end; ++t) {
    const int buf = (t - tile_begin) & 1;
    // ---- S^T = K Q^T: two independent accumulator chains -----------------------------------
    f32x16_t s[2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[mt][i] = 0.0f;
#pragma unroll
    for (int j = 0; j < D / 16; ++j) {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const u32x4_t kk = sm.k[buf][mt * 32 + n][2 * j + h];
        s[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kk), qf[j], s[mt], 0, 0, 0);
      }
    }
    // ---- mask (only tiles that hold a position some row of this wavefront may not see) ----
    {
      const int tpl = sm.tp[buf][lane];
      if (__any(tpl > qpos_min_w)) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int a = 0; a < 4; ++a) {
            const int4 tq = *(const int4*)&sm.tp[buf][mt * 32 + 8 * a + 4 * h];
            if (tq.x > qpos) s[mt][4 * a + 0] = -INFINITY;
            if (tq.y > qpos) s[mt][4 * a + 1] = -INFINITY;
            if (tq.z > qpos) s[mt][4 * a + 2] = -INFINITY;
            if (tq.w > qpos) s[mt][4 * a + 3] = -INFINITY;
          }
      }
    }
    // ---- online softmax --------------------------------------------------------------------
    float mx = fmaxf(s[0][0], s[1][0]);
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(fmaxf(mx, s[0][i]), s[1][i]);
    mx = fmaxf(mx, xor32(mx));
    if (__any(mx > m)) {  // rescale only when some row of the wavefront has a new maximum
      const float m_new = fmaxf(m, mx);
      const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
      const float alpha = fast_exp2((m - m_use) * p.c);
      l *= alpha;
      m = m_new;
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
    }
    const float mc = (m == -INFINITY) ? 0.0f : m * p.c;
    float rs0 = 0.0f, rs1 = 0.0f;
    uint32_t pb[2][8];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float p0 = fast_exp2(fmaf(s[mt][i], p.c, -mc));
        const float p1 = fast_exp2(fmaf(s[mt][i + 1], p.c, -mc));
        rs0 += p0;
        rs1 += p1;
        pb[mt][i >> 1] = pack_bf16(p0, p1);
      }
    l += rs0 + rs1;
    // ---- O^T += V^T P^T ---------------------------------------------------------------------
    const uint16_t* vbase_lds = (const uint16_t*)&sm.v[buf][0][0];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const bf16x8_t pf = as_bf16x8(u32x4_t{pb[mt][4 * j], pb[mt][4 * j + 1], pb[mt][4 * j + 2], pb[mt][4 * j + 3]});
        const int krow = 32 * mt + 16 * j + v_row_off;
#pragma unroll
        for (int dt = 0; dt < D / 32; ++dt) {
          const u32x2_t lo = lds_read_tr16(vbase_lds + krow * (Smem<D>::VCH16 * 8) + 32 * dt + v_col_off);
          const u32x2_t hi = lds_read_tr16(vbase_lds + (krow + 8) * (Smem<D>::VCH16 * 8) + 32 * dt + v_col_off);
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(u32x4_t{lo[0], lo[1], hi[0], hi[1]}), pf, o[dt], 0, 0, 0);
        }
      }
    // ---- stage the next tile ------------------------------------------------------------------
    if (t + 1 < tile_end) {
      ld.commit(st, sm, buf ^ 1, tid);
      if (t + 2 < tile_end) ld.fetch(st, t + 2, tid);
    }
    __syncthreads();
  }

  // ---- epilogue -----------------------------------------------------------------------------
  const float lt = l + xor32(l);
  if (p.num_splits == 1) {
    const float inv = lt > 0.0f ? 1.0f / lt : 0.0f;
    if (row_ok) {
      uint16_t* op = p.o + b * p.o_sb + (int64_t)(kvh * p.G + g) * p.o_sh + (int64_t)qi * p.o_st;
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          u32x2_t w2;
          w2[0] = pack_bf16(o[dt][4 * a] * inv, o[dt][4 * a + 1] * inv);
          w2[1] = pack_bf16(o[dt][4 * a + 2] * inv, o[dt][4 * a + 3] * inv);
          *(u32x2_t*)(op + dt * 32 + 8 * a + 4 * h) = w2;
        }
      if (p.lse && h == 0) p.lse[((int64_t)b * p.q_len + qi) * p.Hq + kvh * p.G + g] = m * p.c + fast_log2(lt);
    }
  } else {
    if (row_ok) {
      const int64_t prow = ((int64_t)split * p.B * p.Hkv + group) * p.R + row;
      float* po = p.part_o + prow * D;
#pragma unroll
      for (int dt = 0; dt < D / 32; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          f32x4_t w4 = {o[dt][4 * a], o[dt][4 * a + 1], o[dt][4 * a + 2], o[dt][4 * a + 3]};
          *(f32x4_t*)(po + dt * 32 + 8 * a + 4 * h) = w4;
        }
      if (h == 0) {
        p.part_ml[prow * 2] = m * p.c;  // -inf if the split saw no visible key
        p.part_ml[prow * 2 + 1] = lt;
      }
    }
  }
}

// Combine the per-split partials of a row: one workgroup of D/4 threads... one thread per 4 d.
template <int D>
__global__ __launch_bounds__(256) void sdpa_prefill_merge_kernel(const PrefillParams p) {
  constexpr int TPR = D / 4;              // threads per row
  constexpr int ROWS = 256 / TPR;         // rows per workgroup
  const int64_t total_rows = (int64_t)p.B * p.Hkv * p.R;
  const int64_t grow = (int64_t)blockIdx.x * ROWS + threadIdx.x / TPR;
  if (grow >= total_rows) return;
  const int dq = threadIdx.x % TPR;
  const int group = (int)(grow / p.R);
  const int row = (int)(grow % p.R);
  const int b = group / p.Hkv, kvh = group % p.Hkv;
  const int qi = row / p.G, g = row % p.G;
  float M = -INFINITY;
  for (int s = 0; s < p.num_splits; ++s) M = fmaxf(M, p.part_ml[((int64_t)s * total_rows + grow) * 2]);
  const float Mu = (M == -INFINITY) ? 0.0f : M;
  float L = 0.0f;
  f32x4_t acc = {0, 0, 0, 0};
  for (int s = 0; s < p.num_splits; ++s) {
    const int64_t pr = (int64_t)s * total_rows + grow;
    const float w = fast_exp2(p.part_ml[pr * 2] - Mu);
    L += p.part_ml[pr * 2 + 1] * w;
    const f32x4_t x = *(const f32x4_t*)(p.part_o + pr * D + dq * 4);
    acc += x * w;
  }
  const float inv = L > 0.0f ? 1.0f / L : 0.0f;
  uint16_t* op = p.o + b * p.o_sb + (int64_t)(kvh * p.G + g) * p.o_sh + (int64_t)qi * p.o_st + dq * 4;
  u32x2_t w2;
  w2[0] = pack_bf16(acc[0] * inv, acc[1] * inv);
  w2[1] = pack_bf16(acc[2] * inv, acc[3] * inv);
  *(u32x2_t*)op = w2;
  if (p.lse && dq == 0) p.lse[((int64_t)b * p.q_len + qi) * p.Hq + kvh * p.G + g] = Mu + fast_log2(L);
}

int pick_splits(const kvx_sdpa_args& a, int m_blocks, int num_tiles) {
  if (a.num_splits > 0) return min(a.num_splits, num_tiles);
  // Aim for about four workgroups per compute unit, at least 8 key tiles per split.
  const int64_t base = (int64_t)a.B * a.Hkv * m_blocks;
  const int target = 4 * num_cus();
  int s = (int)((target + base - 1) / base);
  s = max(1, min(s, num_tiles / 8));
  return max(1, min(s, 64));
}

void fill_params(PrefillParams& p, const kvx_sdpa_args& a) {
  p.q = (const uint16_t*)a.q;
  p.k = a.k;
  p.v = a.v;
  p.k_scale = a.k_scale;
  p.k_zp = a.k_zp;
  p.v_scale = a.v_scale;
  p.v_zp = a.v_zp;
  p.tp = a.token_positions;
  p.o = (uint16_t*)a.o;
  p.lse = a.lse;
  p.B = a.B;
  p.Hq = a.Hq;
  p.Hkv = a.Hkv;
  p.G = a.Hq / a.Hkv;
  p.q_len = a.q_len;
  p.kv_len = a.kv_len;
  p.R = a.q_len * p.G;
  p.input_pos = a.input_pos;
  p.num_tiles = (a.kv_len + BN - 1) / BN;
  p.m_blocks = (p.R + BM - 1) / BM;
  p.num_splits = pick_splits(a, p.m_blocks, p.num_tiles);
  p.tiles_per_split = (p.num_tiles + p.num_splits - 1) / p.num_splits;
  p.num_splits = (p.num_tiles + p.tiles_per_split - 1) / p.tiles_per_split;
  p.c = a.sm_scale * kLog2e;
  p.q_sb = a.q_stride_b; p.q_sh = a.q_stride_h; p.q_st = a.q_stride_t;
  p.k_sb = a.k_stride_b; p.k_sh = a.k_stride_h; p.k_st = a.k_stride_t;
  p.v_sb = a.v_stride_b; p.v_sh = a.v_stride_h; p.v_st = a.v_stride_t;
  p.o_sb = a.o_stride_b; p.o_sh = a.o_stride_h; p.o_st = a.o_stride_t;
  p.qs_sb = a.qs_stride_b; p.qs_sh = a.qs_stride_h;
  p.tp_sb = a.tp_stride_b; p.tp_sh = a.tp_stride_h;
  p.part_o = nullptr;
  p.part_ml = nullptr;
}

size_t partial_bytes(const PrefillParams& p, int D) {
  if (p.num_splits <= 1) return 0;
  const size_t rows = (size_t)p.num_splits * p.B * p.Hkv * p.R;
  return rows * (size_t)D * 4 + rows * 2 * 4;
}

template <int D, bool U8>
int launch_t(PrefillParams& p, hipStream_t st) {
  dim3 grid(p.B * p.Hkv, p.m_blocks, p.num_splits);
  hipLaunchKernelGGL((sdpa_prefill_kernel<D, U8>), grid, dim3(NTHREADS), 0, st, p);
  KVX_HIP(hipGetLastError());
  if (p.num_splits > 1) {
    constexpr int ROWS = 256 / (D / 4);
    const int64_t total_rows = (int64_t)p.B * p.Hkv * p.R;
    hipLaunchKernelGGL((sdpa_prefill_merge_kernel<D>), dim3((unsigned)((total_rows + ROWS - 1) / ROWS)), dim3(256), 0, st, p);
    KVX_HIP(hipGetLastError());
  }
  return KVX_OK;
}

}  // namespace

size_t sdpa_prefill_workspace(const kvx_sdpa_args& a) {
  PrefillParams p;
  fill_params(p, a);
  return partial_bytes(p, a.D);
}

int launch_sdpa_prefill(const kvx_sdpa_args& a, hipStream_t st) {
  PrefillParams p;
  fill_params(p, a);
  const size_t need = partial_bytes(p, a.D);
  if (need) {
    KVX_REQUIRE(a.workspace && a.workspace_bytes >= need, KVX_ERR_WORKSPACE,
                "kvx_sdpa_prefill: workspace of %zu bytes needed, %zu given", need, a.workspace_bytes);
    const size_t rows = (size_t)p.num_splits * p.B * p.Hkv * p.R;
    p.part_o = (float*)a.workspace;
    p.part_ml = p.part_o + rows * (size_t)a.D;
  }
  const bool u8 = a.kv_dtype == KVX_KV_U8;
  if (a.D == 128) return u8 ? launch_t<128, true>(p, st) : launch_t<128, false>(p, st);
  if (a.D == 64) return u8 ? launch_t<64, true>(p, st) : launch_t<64, false>(p, st);
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_sdpa_prefill: head size %d not in {64, 128}", a.D);
}

}  // namespace kvx
