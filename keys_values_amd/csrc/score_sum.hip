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

// Q tile in LDS: [row][16-byte chunk], rows unpadded (what the global -> LDS transfer writes: a wavefront
// instruction fills 1024 contiguous bytes), chunk c of row r stored at position c ^ swz(r). The operand reads
// (ds_read_b128, 16 consecutive rows and the same chunk per phase) then touch every bank once.
template <int CPR>
__device__ __forceinline__ int swz(int r) { return CPR >= 16 ? (r & 15) : ((r >> 1) & 7); }

template <int D>
struct alignas(16) Smem {
  static constexpr int CPR = D / 8;  // 16-byte chunks per row
  u32x4_t q[2][BQ][CPR];
  float lse[2][BQ];     // a tile's log-sum-exps are in registers before the barrier that frees its Q buffer
  int32_t qpos[4][BQ];  // read through the whole step (only by tiles that need the mask): a ring of four
};

// Streams the packed query rows (row r = query r / G, head r % G) of one (batch, KV head) pair into LDS, tile by
// tile, with global -> LDS transfers: no registers hold the rows on their way. Wavefront w issues instructions
// w, w + W, ... of the CPR that make a tile (RPW = 64 / CPR rows each); lane l of instruction i fills LDS position
// l % CPR of row i RPW + l / CPR, so it fetches the chunk that belongs there under the swizzle. Addresses are a
// uniform base plus a 32-bit byte offset per lane (the host checks the range). Wavefront 0 also fetches the rows'
// log-sum-exps (4 bytes per lane) and writes their positions.
//   issue_steady: G divides the tile height and the tile is full. Every row keeps its head and moves by BQ / G
//     queries from tile to tile: the base advances by scalar adds and the lane offsets stay.
//   issue: any tile. The offsets are formed per lane from the row's (query, head); rows past the end re-read the
//     last valid row, and land() overwrites their log-sum-exp with +inf, so their weight is exactly zero.
template <int D, int W>
struct QLoader {
  static constexpr int CPR = D / 8;
  static constexpr int RPW = 64 / CPR;
  static constexpr int NI = CPR / W;      // transfers per wavefront and tile
  static constexpr int TILE_BYTES = BQ * CPR * 16;
  const char* qbase;   // (b, first head of the group)
  const char* lbase;   // lse + b * q_len * Hq + kvh * G
  const char* qtile;   // issue_steady: qbase advanced to the tile it fetches next
  const char* ltile;   // likewise for the log-sum-exps
  uint32_t voff0[NI];  // issue_steady: byte offset of this lane's chunk of instruction i relative to qtile
  uint32_t loff0;      // likewise for the log-sum-exp of row `lane`
  int qpv;             // likewise the position of row `lane`
  uint32_t cb[NI];     // byte offset of the chunk inside a row
  int rin[NI];         // row inside the tile
  uint32_t q_shb, q_stb, qstep, lstep;
  float inv_g;         // 1 / G: (int)((r + 0.5f) * inv_g) == r / G for the small r of a tile
  int G, R, Hq, input_pos, dq, dg, wave, lane;
  int q0, g0;          // (query, head) of the first row of the next tile to fetch
  uint32_t lds_qw, lds_lse, lds_qpos;
  int next_row0;       // first row of the next tile to fetch

  // steady_first: index (counted from row_start) of the first tile issue_steady will be asked for
  __device__ __forceinline__ void init(const ScoreParams& p, Smem<D>& sm, int b, int kvh, int tid, int row_start, int steady_first) {
    wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    lane = tid & 63;
    G = p.G; R = p.R; Hq = p.Hq; input_pos = p.input_pos;
    q_shb = (uint32_t)p.q_sh * 2u; q_stb = (uint32_t)p.q_st * 2u;
    qbase = (const char*)(p.q + b * p.q_sb + (int64_t)(kvh * p.G) * p.q_sh);
    lbase = (const char*)(p.lse + (int64_t)b * p.q_len * p.Hq + kvh * p.G);
    dq = BQ / G; dg = BQ % G;
    inv_g = 1.0f / (float)G;
    qstep = (uint32_t)dq * q_stb;
    lstep = (uint32_t)(dq * Hq) * 4u;
    q0 = row_start / G;
    g0 = row_start % G;
    const int qs = q0 + steady_first * dq;        // dg == 0: row_start is a multiple of BQ, hence of G
    qtile = qbase + (uint64_t)qs * q_stb;
    ltile = lbase + (uint64_t)(qs * Hq) * 4u;
    qpv = input_pos + qs + lane / G;
    lds_qw = __builtin_amdgcn_readfirstlane(lds_addr_of(&sm.q[0][0][0]) + (uint32_t)(wave * 1024));
    lds_lse = __builtin_amdgcn_readfirstlane(lds_addr_of(&sm.lse[0][0]));
    lds_qpos = lds_addr_of(&sm.qpos[0][0]) + (uint32_t)(lane * 4);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      rin[i] = (wave + W * i) * RPW + lane / CPR;
      cb[i] = (uint32_t)(((lane % CPR) ^ swz<CPR>(rin[i])) * 16);
      voff0[i] = (uint32_t)(rin[i] % G) * q_shb + (uint32_t)(rin[i] / G) * q_stb + cb[i];
    }
    loff0 = (uint32_t)((lane / G) * Hq + lane % G) * 4u;
    next_row0 = row_start;
  }

  template <int BUF, int I = 0>
  __device__ __forceinline__ void dma_q_steady() {
    dma16_at<(uint32_t)(BUF * TILE_BYTES + W * I * 1024)>(qtile, voff0[I], lds_qw);
    if constexpr (I + 1 < NI) dma_q_steady<BUF, I + 1>();
  }
  template <int BUF>
  __device__ __forceinline__ void issue_steady(Smem<D>& sm, int ring) {
    dma_q_steady<BUF>();
    if (wave == 0) {
      dma4_at<(uint32_t)(BUF * BQ * 4)>(ltile, loff0, lds_lse);
      sm.qpos[ring][lane] = qpv;
      qpv += dq;
    }
    qtile += qstep;
    ltile += lstep;
    q0 += dq;
    next_row0 += BQ;
  }

  // start the transfers of the next tile into Q / lse buffer `buf` and position buffer `ring`
  __device__ __forceinline__ void issue(Smem<D>& sm, int buf, int ring) {
    const int row0 = next_row0;
    const int rl = R - 1;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int r = min(g0 + rin[i] + q0 * G, rl) - q0 * G;  // row relative to (q0, head 0), clamped to the last valid row
      const int dqi = (int)(((float)r + 0.5f) * inv_g);         // r / G, r < G + BQ
      dma16(qbase, (uint32_t)(r - dqi * G) * q_shb + (uint32_t)(q0 + dqi) * q_stb + cb[i], lds_qw + (uint32_t)(buf * TILE_BYTES + W * i * 1024));
    }
    if (wave == 0) {
      const bool ok = row0 + lane < R;
      const int r = min(g0 + lane + q0 * G, rl) - q0 * G;
      const int dqi = (int)(((float)r + 0.5f) * inv_g);
      dma4(lbase, (uint32_t)((q0 + dqi) * Hq + (r - dqi * G)) * 4u, lds_lse + (uint32_t)(buf * BQ * 4));
      sm.qpos[ring][lane] = ok ? input_pos + q0 + dqi : INT_MAX;
    }
    q0 += dq;
    g0 += dg;
    if (g0 >= G) {
      g0 -= G;
      q0 += 1;
    }
    next_row0 = row0 + BQ;
  }

  // after s_waitcnt vmcnt(0), before the barrier that publishes the tile whose first row is row0
  __device__ __forceinline__ void land(Smem<D>& sm, int row0, int buf) const {
    if (row0 + BQ > R && wave == 0 && row0 + lane >= R) sm.lse[buf][lane] = INFINITY;  // exp2(... - inf) = 0
  }
};

// QSPLIT: the query rows are split over blockIdx.z (short caches that would otherwise leave compute units
// idle); every split writes its sums to p.part and a second kernel adds them in a fixed order.
//
// The kernel is bound by the number of instructions a wavefront issues per tile (two wavefronts per SIMD issue
// about one instruction per ten cycles each, whatever its kind), so the tile loop comes in three forms: tiles that
// need the position mask and tiles that do not, each unrolled by two with every LDS address an immediate and the
// transfers of the tile after next sent without bounds checks ("steady"), and a general form for the last tiles.
template <int D, int KV, int W, bool QSPLIT>
__global__ __launch_bounds__(64 * W, D <= 128 ? 2 : 1) void score_sum_kernel(const ScoreParams p) {
  constexpr int BK = NW * W;  // keys per workgroup
  constexpr bool F16 = kv_elem_f16(KV);  // element type of q and k
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
        if constexpr (kv_is_u4(KV)) {  // chunk 2j + h of the row: one nibble of 8 bytes
          cc = ok ? *(const u32x2_t*)(kp + u4_byte_off<D>(2 * j + h)) : u32x2_t{0, 0};
          cc = u4_codes(cc, u4_shift<D>(2 * j + h));
        } else {
          cc = ok ? *(const u32x2_t*)(kp + 16 * j + 8 * h) : u32x2_t{0, 0};
        }
        kf[nt][j] = dequant_words<F16>(cc[0], cc[1], zp, sc);
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
  // Steps [0, t_steady) are steady: G divides the tile height and tiles t + 1 and t + 2 exist and are full.
  // Steps [0, t_masked) need the mask: the first query position of tile t, input_pos + (tbase + t) BQ / G, is below
  // the largest key position of this wavefront. Both are even, so the buffer index stays a compile-time constant.
  const int nfull = min(num_qt, p.R / BQ - tbase);
  const int t_steady = (BQ % p.G == 0) ? (max(nfull - 2, 0) & ~1) : 0;
  int t_masked;
  {
    const int64_t need = (int64_t)max(min(tpmax, p.input_pos + p.q_len) - p.input_pos, 0) * p.G;  // rows whose position is below tpmax
    const int64_t tiles = (need + BQ - 1) / BQ - tbase;
    t_masked = (int)max((int64_t)0, min(tiles, (int64_t)num_qt));
    t_masked = min((t_masked + 1) & ~1, t_steady);
  }
  QLoader<D, W> ld;
  ld.init(p, sm, b, kvh, tid, tbase * BQ, 2);
  // LDS byte offsets of this lane's Q fragments (A operand): row mt 32 + n, chunk 2 j + h at position chunk ^ swz(row)
  constexpr int CPR = D / 8;
  uint32_t qa[D / 16];
#pragma unroll
  for (int j = 0; j < D / 16; ++j) qa[j] = (uint32_t)((n * CPR + ((2 * j + h) ^ swz<CPR>(n))) * 16);

  // The Q fragments of a block (32 query rows, A operand) and the rows' log-sum-exps are requested together, ahead
  // of the block's first matrix instruction: the reads then have the previous block's tail to arrive in. BUF is a
  // compile-time constant, so every read is one address register plus an immediate offset.
  auto load_q = [&](u32x4_t (&qq)[D / 16], auto buf_tag, auto mt_tag) {
    constexpr int BUF = decltype(buf_tag)::value, MT = decltype(mt_tag)::value;
    const char* qb = (const char*)&sm.q[BUF][MT * 32][0];
#pragma unroll
    for (int j = 0; j < D / 16; ++j) qq[j] = *(const u32x4_t*)(qb + qa[j]);
  };
  // accumulator rows of a lane are 8 a + 4 h + (0..3)
  auto load_lse = [&](f32x4_t (&ls)[4], auto buf_tag, auto mt_tag) {
    constexpr int BUF = decltype(buf_tag)::value, MT = decltype(mt_tag)::value;
#pragma unroll
    for (int a = 0; a < 4; ++a) ls[a] = *(const f32x4_t*)&sm.lse[BUF][MT * 32 + 8 * a + 4 * h];
  };
  // S block = 32 query rows x 64 keys, K in registers
  auto mfma_block = [&](f32x16_t (&s)[2], const u32x4_t (&qq)[D / 16]) {
#pragma unroll
    for (int j = 0; j < D / 16; ++j) {
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        if (j == 0) {
          const f32x16_t zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          s[nt] = mfma_32x32x16<F16>(qq[j], kf[nt][j], zero);
        } else {
          s[nt] = mfma_32x32x16<F16>(qq[j], kf[nt][j], s[nt]);
        }
      }
    }
  };
  // p = exp2(c S - lse) summed over the block's rows
  auto valu_block = [&](auto mask_tag, const f32x16_t (&s)[2], const f32x4_t (&ls)[4], int ring, int mt) {
    constexpr bool MASK = decltype(mask_tag)::value;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      int4 qp = {0, 0, 0, 0};
      if constexpr (MASK) qp = *(const int4*)&sm.qpos[ring][mt * 32 + 8 * a + 4 * h];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        float e0 = fast_exp2(fmaf(s[nt][4 * a + 0], p.c, -ls[a][0]));
        float e1 = fast_exp2(fmaf(s[nt][4 * a + 1], p.c, -ls[a][1]));
        float e2 = fast_exp2(fmaf(s[nt][4 * a + 2], p.c, -ls[a][2]));
        float e3 = fast_exp2(fmaf(s[nt][4 * a + 3], p.c, -ls[a][3]));
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
  // one matrix instruction, then its share of the other block's vector work (6 or 10 instructions per matrix
  // instruction, 2 of them transcendental)
  auto interleave = [&](auto mask_tag) {
    constexpr bool MASK = decltype(mask_tag)::value;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      if constexpr (MASK) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // the positions of rows 8 a .. 8 a + 7
#pragma unroll
      for (int i = 0; i < (D / 16) / 2; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, MASK ? 8 * 16 / (2 * (D / 16)) : 4 * 16 / (2 * (D / 16)), 0);
        __builtin_amdgcn_sched_group_barrier(0x400, 2 * 16 / (2 * (D / 16)), 0);
      }
    }
  };

  // Keeps a half step's work in that half: without a use here the optimiser moves the exponentials of several
  // half steps below the matrix instructions of the next ones (out of their shadow, and every block's scores then
  // need registers of their own).
  auto pin = [&](f32x16_t (&s)[2]) {
    asm volatile("" : "+v"(s[0]), "+v"(s[1]), "+v"(wacc[0]), "+v"(wacc[1]));
  };
  constexpr std::integral_constant<int, 0> I0{};
  constexpr std::integral_constant<int, 1> I1{};
  ld.issue(sm, 0, 0);
  if (num_qt > 1) ld.issue(sm, 1, 1);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the K fragments and the first tiles have arrived
  ld.land(sm, tbase * BQ, 0);
  if (num_qt > 1) ld.land(sm, (tbase + 1) * BQ, 1);
  __syncthreads();
  f32x16_t sa[2], sb[2];  // blocks 0 and 1 of the current tile
  u32x4_t qq[D / 16];
  load_q(qq, I0, I0);
  mfma_block(sa, qq);

  // Software pipeline: the matrix work of one block runs under the vector work of the block before.
  // Tile t + 2 is requested right behind the barrier of step t (the buffers of tile t are free from there on: its
  // Q rows have been multiplied and its log-sum-exps are in registers), has the rest of that step and the first
  // half of the next to arrive, and is published by the barrier of step t + 1.
  auto step = [&](auto mask_tag, auto steady_tag, auto buf_tag, int t) {
    constexpr bool STEADY = decltype(steady_tag)::value;
    constexpr int BUF = decltype(buf_tag)::value;
    constexpr std::integral_constant<int, BUF ^ 1> NEXT{};
    const int ring = t & 3;
    const bool more = STEADY || t + 1 < num_qt;
    f32x4_t ls[4];
    load_q(qq, buf_tag, I1);
    load_lse(ls, buf_tag, I0);
    __builtin_amdgcn_sched_barrier(0);
    mfma_block(sb, qq);
    valu_block(mask_tag, sa, ls, ring, 0);
    interleave(mask_tag);
    pin(sb);
    __builtin_amdgcn_sched_barrier(0);
    load_lse(ls, buf_tag, I1);  // into registers before the barrier that hands the buffer to tile t + 2
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's part of tile t + 1 has landed
    if constexpr (!STEADY) {
      if (more) ld.land(sm, (tbase + t + 1) * BQ, BUF ^ 1);
    }
    __syncthreads();
    if constexpr (STEADY) {
      ld.template issue_steady<BUF>(sm, (t + 2) & 3);
    } else {
      if (t + 2 < num_qt) ld.issue(sm, BUF, (t + 2) & 3);
    }
    if (more) {
      load_q(qq, NEXT, I0);
      __builtin_amdgcn_sched_barrier(0);
      mfma_block(sa, qq);
      valu_block(mask_tag, sb, ls, ring, 1);
      interleave(mask_tag);
      pin(sa);
      __builtin_amdgcn_sched_barrier(0);
    } else {
      valu_block(mask_tag, sb, ls, ring, 1);
    }
  };
  constexpr std::true_type YES{};
  constexpr std::false_type NO{};
  int t = 0;
  for (; t < t_masked; t += 2) {
    step(YES, YES, I0, t);
    step(YES, YES, I1, t + 1);
  }
  for (; t < t_steady; t += 2) {
    step(NO, YES, I0, t);
    step(NO, YES, I1, t + 1);
  }
  // the last tiles (and all of them when G does not divide the tile height): masked whether they need it or not
  for (; t + 1 < num_qt; t += 2) {
    step(YES, NO, I0, t);
    step(YES, NO, I1, t + 1);
  }
  if (t < num_qt) step(YES, NO, I0, t);

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
  // the query rows are fetched at a uniform base plus a 32-bit byte offset per lane
  {
    const int64_t G = a.Hq / a.Hkv;
    KVX_REQUIRE(a.q_stride_h >= 0 && a.q_stride_t >= 0 && ((G - 1) * a.q_stride_h + (int64_t)(a.q_len - 1) * a.q_stride_t + a.D) * 2 < (1ll << 32),
                KVX_ERR_UNSUPPORTED, "kvx_score_sum: the query rows of one (batch, KV head) pair must span less than 4 GiB (strides %lld / %lld)",
                (long long)a.q_stride_h, (long long)a.q_stride_t);
  }
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
#define KVX_SCORE_SUM_CASE(KV) \
  case KV: \
    return a.D == 256 ? launch_t<256, KV>(p, pl.splits, st) : a.D == 128 ? launch_t<128, KV>(p, pl.splits, st) : launch_t<64, KV>(p, pl.splits, st);
  if (a.D == 256 || a.D == 128 || a.D == 64) {
    switch (a.kv_dtype) {
      KVX_SCORE_SUM_CASE(KVX_KV_BF16)
      KVX_SCORE_SUM_CASE(KVX_KV_F16)
      KVX_SCORE_SUM_CASE(KVX_KV_U8)
      KVX_SCORE_SUM_CASE(KVX_KV_U4)
      KVX_SCORE_SUM_CASE(KVX_KV_U8_F16)
      KVX_SCORE_SUM_CASE(KVX_KV_U4_F16)
    }
  }
#undef KVX_SCORE_SUM_CASE
  return set_error(KVX_ERR_UNSUPPORTED, "kvx_score_sum: head size %d not in {64, 128, 256}", a.D);
}

}  // namespace kvx
