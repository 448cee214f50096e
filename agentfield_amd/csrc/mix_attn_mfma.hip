// Masked (causal / chunk-local / banded) paged prefill attention on the
// matrix cores, bf16 storage, for head sizes up to 128 that need not be a
// power of two.  Scores, mask, softmax statistics and the output accumulator
// are fp32; Q.K^T and P.V run as MFMA 16x16x32 bf16.
//
// Workgroup = 64 consecutive chunk rows of one sequence x one query head;
// wave w owns rows 16w..16w+15.  Key/value tiles of 64 positions are staged
// once per workgroup through LDS: K row-major (rows padded by 16 B), V
// transposed [d][token] with token pairs packed into 32-bit writes, the
// wave's probabilities round-trip through a private LDS tile to turn the
// MFMA C layout into an A fragment.  Head sizes are zero-padded to the
// template extent (DKC*32 for q/k, DVT*16 for v).  Only key tiles that
// intersect the rows' visible range are visited: for chunk-local attention
// that is at most chunk/64 + 1 tiles per workgroup.
//
// Fragment layouts of v_mfma_f32_16x16x32_bf16 (64-lane wave):
//   A: lane holds A[m = lane&15][k = (lane>>4)*8 + j], j = 0..7
//   B: lane holds B[k = (lane>>4)*8 + j][n = lane&15]
//   C: lane reg r holds C[m = (lane>>4)*4 + r][n = lane&15]
#include "common.h"
#include "mix_attn.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

__device__ __forceinline__ bf16x8 as_bf16x8(s16x8 v) {
  union { s16x8 s; bf16x8 b; } u;
  u.s = v;
  return u.b;
}

// 8 consecutive bf16 starting at element e0 of a row of n valid elements;
// elements >= n read as zero.  VEC: rows and e0 are 16-byte aligned and n is
// a multiple of 8, so a group is either fully inside or fully outside.
template <bool VEC>
__device__ __forceinline__ s16x8 load8(const u16* row, int e0, int n) {
  s16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
  if (VEC) {
    if (e0 < n) v = *reinterpret_cast<const s16x8*>(row + e0);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (e0 + j < n) v[j] = (short)row[e0 + j];
  }
  return v;
}

// Stage one tile of KT keys: K rows row-major into k_lds, V rows transposed into
// v_lds ([d][token], token pairs packed into 32-bit writes).  The page walk
// is done once per key (row_lds[tok] = row index in the pages, -1 for keys
// past `last`), so the tile's loads depend on nothing but LDS and are issued
// back to back.
template <int DKC, int DVT, bool VEC, int NT = 256, int KT = 64>
__device__ __forceinline__ void stage_kv_tile(
    u16* k_lds, u16* v_lds, i32* row_lds, const u16* __restrict__ kc,
    const u16* __restrict__ vc, const i32* __restrict__ btr, int kv0, int last,
    int G, int g, int page, int dk, int dv, i64 ldv) {
  constexpr int KS = DKC * 32 + 8;
  constexpr int VS = KT + 8;
  constexpr int TP = KT / 2;                  // token pairs
  if (threadIdx.x < KT) {
    const int j = kv0 + threadIdx.x;
    row_lds[threadIdx.x] =
        j <= last ? (btr[j / page] * G + g) * page + (j % page) : -1;
  }
  __syncthreads();
  constexpr int KIT = (KT * DKC * 4 + NT - 1) / NT;
#pragma unroll
  for (int it = 0; it < KIT; ++it) {
    const int i = it * NT + threadIdx.x;
    if (i >= KT * DKC * 4) break;
    const int tok = i / (DKC * 4), e0 = (i % (DKC * 4)) * 8;
    const int row = row_lds[tok];
    s16x8 v8 = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row >= 0) v8 = load8<VEC>(kc + (size_t)row * dk, e0, dk);
    *reinterpret_cast<s16x8*>(k_lds + tok * KS + e0) = v8;
  }
  constexpr int VIT = (TP * DVT * 2 + NT - 1) / NT;
#pragma unroll
  for (int it = 0; it < VIT; ++it) {
    const int i = it * NT + threadIdx.x;
    if (i >= TP * DVT * 2) break;
    const int tp = i % TP, e0 = (i / TP) * 8;
    const int ra = row_lds[tp * 2], rb = row_lds[tp * 2 + 1];
    s16x8 a = {0, 0, 0, 0, 0, 0, 0, 0}, c8 = a;
    if (ra >= 0) a = load8<VEC>(vc + (size_t)ra * ldv, e0, dv);
    if (rb >= 0) c8 = load8<VEC>(vc + (size_t)rb * ldv, e0, dv);
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      const uint32_t packed = (uint32_t)(unsigned short)a[jj] |
                              ((uint32_t)(unsigned short)c8[jj] << 16);
      *reinterpret_cast<uint32_t*>(v_lds + (e0 + jj) * VS + tp * 2) = packed;
    }
  }
}

// NH = 2: two query heads of one K/V group per workgroup (eight waves), so a
// staged tile serves both and one head's LDS / MFMA waits hide behind the
// other's VALU work.  KT: keys per staged tile (64, or 32 where two heads'
// 64-key tiles would not fit in LDS).
template <int DKC, int DVT, bool VEC, int NH, int KT>
__device__ __forceinline__ void attn_prefill_mfma_body(
    u16* __restrict__ out, const u16* __restrict__ q,
    const u16* __restrict__ kc, const u16* __restrict__ vc,
    const i32* __restrict__ bt, const i32* __restrict__ cu,
    const i32* __restrict__ q_start, const i32* __restrict__ tile_seq,
    const i32* __restrict__ tile_q0, float scale, int H, int G, int dk, int dv,
    int page, int maxp, int chunk, int window, i64 ldq, const AttnExtra& ex) {
  constexpr int KS = DKC * 32 + 8;   // K row stride in LDS (elements)
  constexpr int VS = KT + 8;         // V^T / P row stride (KT tokens + pad)
  constexpr int NST = KT / 16;       // 16-key sub-tiles
  constexpr int NHF = KT / 32;       // 32-key halves of P V
  __shared__ u16 k_lds[KT * KS];
  __shared__ u16 v_lds[DVT * 16 * VS];
  __shared__ u16 p_lds[NH * 4 * 16 * VS];
  __shared__ float bias_lds[NH * 128];  // distance bias of this tile's distances
  __shared__ i32 row_lds[KT];        // page row of every key of the tile

  const int hsel = threadIdx.x >> 8;           // which of the NH heads
  const int tile = blockIdx.x, h = blockIdx.y * NH + hsel;
  const int g = h / (H / G);
  const int wid = (threadIdx.x >> 6) & 3, lane = threadIdx.x & 63;
  const int b = tile_seq[tile];
  const int r0 = cu[b];
  const int len = cu[b + 1] - r0;
  const int q0 = tile_q0[tile];                // first chunk row of the tile
  const int nrows = min(64, len - q0);
  const int p0 = q_start[b] + q0;              // position of the first row
  const int p_last = p0 + nrows - 1;
  const i32* btr = bt + (size_t)b * maxp;

  // visible key range of the whole tile: row p0 reaches back the farthest
  int lo = 0;
  if (chunk > 0) lo = (p0 / chunk) * chunk;
  if (window > 0) lo = max(lo, p0 - window + 1);

  // this wave's rows
  const int wrow0 = wid * 16;
  const bool wave_live = wrow0 < nrows;
  const int wp0 = p0 + wrow0;                              // first position
  const int wp_last = min(p0 + wrow0 + 15, p_last);        // last position

  s16x8 q_frag[DKC];
  {
    const int row = min(q0 + wrow0 + (lane & 15), len - 1);
    const u16* qr = q + (size_t)(r0 + row) * ldq + (size_t)h * dk;
#pragma unroll
    for (int c = 0; c < DKC; ++c)
      q_frag[c] = load8<VEC>(qr, c * 32 + (lane >> 4) * 8, dk);
  }
  float m[4], l[4];
  f32x4 o_acc[DVT];
  // the sink enters as a key of score sink[h] and value 0 seen by every row
  const float m0 = ex.sink ? ex.sink[h] : AF_NEG_INF;
#pragma unroll
  for (int r = 0; r < 4; ++r) { m[r] = m0; l[r] = ex.sink ? 1.f : 0.f; }
#pragma unroll
  for (int dt = 0; dt < DVT; ++dt) o_acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  u16* pw = p_lds + (hsel * 4 + wid) * 16 * VS;
  const float r1 = ex.r1 ? ex.r1[h] : 0.f, r2 = ex.r1 ? ex.r2[h] : 0.f;
  const float inv_cap = ex.cap > 0.f ? 1.0f / ex.cap : 0.f;

  // always-visible leading keys that lie in front of the window are walked
  // first, in whole tiles from key 0; the window's tiles follow from b0
  const int nfirst = (ex.first > 0 && lo > 0) ? min(ex.first, lo) : 0;
  const int a_end = (nfirst + KT - 1) / KT * KT;
  const int b0 = max(lo, a_end);
  for (int kv0 = nfirst > 0 ? 0 : lo; kv0 <= p_last;
       kv0 = (kv0 < a_end && kv0 + KT >= a_end) ? b0 : kv0 + KT) {
    __syncthreads();   // fragment reads of the previous tile are done
    stage_kv_tile<DKC, DVT, VEC, 256 * NH, KT>(k_lds, v_lds, row_lds, kc, vc,
                                               btr, kv0, p_last, G, g, page,
                                               dk, dv, ex.ldv);
    // distance bias for every distance between a row and a key of the tile:
    // entry i is distance i + (p0 - kv0 - (KT-1)); keys ahead of a row are masked
    if (ex.r1 && (threadIdx.x & 255) < 63 + KT) {     // each head its own table
      const int dist = (int)(threadIdx.x & 255) + p0 - kv0 - (KT - 1);
      bias_lds[hsel * 128 + (threadIdx.x & 255)] =
          dist > 0 ? attn_dist_bias(r1, r2, dist) : 0.f;
    }
    __syncthreads();
    // keys of this tile that any row of the wave may see
    if (!wave_live || kv0 > wp_last) continue;
    if (window > 0 && kv0 + KT - 1 <= wp0 - window && kv0 >= ex.first) continue;

    // ---- S = Q K^T: 16-key sub-tiles ----
    f32x4 s_acc[NST];
#pragma unroll
    for (int st = 0; st < NST; ++st) {
      s_acc[st] = f32x4{0.f, 0.f, 0.f, 0.f};
      const u16* krow = k_lds + (st * 16 + (lane & 15)) * KS + (lane >> 4) * 8;
#pragma unroll
      for (int c = 0; c < DKC; ++c) {
        const s16x8 kf = *reinterpret_cast<const s16x8*>(krow + c * 32);
        s_acc[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            as_bf16x8(q_frag[c]), as_bf16x8(kf), s_acc[st], 0, 0, 0);
      }
    }
    // ---- mask + online softmax; reg r is row (lane>>4)*4 + r ----
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int p = wp0 + (lane >> 4) * 4 + r;
      int rlo = 0;
      if (chunk > 0) rlo = (p / chunk) * chunk;
      if (window > 0) rlo = max(rlo, p - window + 1);
      float sr[NST];
      float tmax = AF_NEG_INF;
#pragma unroll
      for (int st = 0; st < NST; ++st) {
        const int j = kv0 + st * 16 + (lane & 15);
        float sv = s_acc[st][r] * scale;
        if (ex.cap > 0.f) sv = attn_softcap_fast(sv, inv_cap, ex.cap);
        if (ex.r1) sv -= bias_lds[hsel * 128 + (p - p0) - (j - kv0) + KT - 1];
        sr[st] = (j <= p && (j >= rlo || j < ex.first)) ? sv : AF_NEG_INF;
        tmax = fmaxf(tmax, sr[st]);
      }
      tmax = group16_max_f32(tmax);
      const float mn = fmaxf(m[r], tmax);
      const float corr = (m[r] <= AF_NEG_INF) ? 0.f : __expf(m[r] - mn);
      float psum = 0.f;
#pragma unroll
      for (int st = 0; st < NST; ++st) {
        sr[st] = (sr[st] <= AF_NEG_INF) ? 0.f : __expf(sr[st] - mn);
        psum += sr[st];
        s_acc[st][r] = sr[st];
      }
      l[r] = l[r] * corr + group16_sum_f32(psum);
      m[r] = mn;
#pragma unroll
      for (int dt = 0; dt < DVT; ++dt) o_acc[dt][r] *= corr;
    }
    // ---- P: C layout -> A fragments through the wave's LDS tile ----
#pragma unroll
    for (int st = 0; st < NST; ++st)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        pw[((lane >> 4) * 4 + r) * VS + st * 16 + (lane & 15)] = f2bf(s_acc[st][r]);
    __builtin_amdgcn_wave_barrier();
    s16x8 pf[NHF];
#pragma unroll
    for (int hf = 0; hf < NHF; ++hf)
      pf[hf] = *reinterpret_cast<const s16x8*>(pw + (lane & 15) * VS + hf * 32 + (lane >> 4) * 8);
    __builtin_amdgcn_wave_barrier();
    // ---- O += P V ----
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt) {
      const u16* vrow = v_lds + (dt * 16 + (lane & 15)) * VS + (lane >> 4) * 8;
#pragma unroll
      for (int hf = 0; hf < NHF; ++hf) {
        const s16x8 vf = *reinterpret_cast<const s16x8*>(vrow + hf * 32);
        o_acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            as_bf16x8(pf[hf]), as_bf16x8(vf), o_acc[dt], 0, 0, 0);
      }
    }
  }

  if (!wave_live) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = q0 + wrow0 + (lane >> 4) * 4 + r;
    if (row >= len) continue;
    const float inv = l[r] > 0.f ? 1.0f / l[r] : 0.f;
    u16* op = out + ((size_t)(r0 + row) * H + h) * dv;
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt) {
      const int d = dt * 16 + (lane & 15);
      if (d < dv) op[d] = f2bf(o_acc[dt][r] * inv);
    }
  }
}

#define AF_APM_PARAMS                                                          \
    u16* __restrict__ out, const u16* __restrict__ q,                          \
    const u16* __restrict__ kc, const u16* __restrict__ vc,                    \
    const i32* __restrict__ bt, const i32* __restrict__ cu,                    \
    const i32* __restrict__ q_start, const i32* __restrict__ tile_seq,         \
    const i32* __restrict__ tile_q0, float scale, int H, int G, int dk, int dv,\
    int page, int maxp, int chunk, int window, i64 ldq, AttnExtra ex
#define AF_APM_ARGS                                                            \
    out, q, kc, vc, bt, cu, q_start, tile_seq, tile_q0, scale, H, G, dk, dv,   \
    page, maxp, chunk, window, ldq, ex

template <int DKC, int DVT, bool VEC, int NH, int KT = 64>
__global__ void __launch_bounds__(256 * NH) attn_prefill_mfma_kernel(AF_APM_PARAMS) {
  attn_prefill_mfma_body<DKC, DVT, VEC, NH, KT>(AF_APM_ARGS);
}

// The widest instance keeps 16 x 512 output accumulators and an 18-fragment
// query per wave: two waves per SIMD (the eight waves of one workgroup) is all
// a CU can hold of it, so it may use their full register share.
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
attn_prefill_mfma_wide_pair_kernel(AF_APM_PARAMS) {
  attn_prefill_mfma_body<18, 32, true, 2, 32>(AF_APM_ARGS);
}

// ------------------------------------------------ single rows, many heads
// One token's query heads of a K/V group as the rows of the MFMA tiles: the
// case of decode steps when many heads share one K/V head (16 heads on one
// latent row are exactly one 16-row tile), where a lane-per-key walk spends
// its time on H dot products per key.  Workgroup = (token, K/V group x block
// of 16 heads, key split); all four waves hold the block's queries.  Per
// 64-key tile wave w takes keys 16w..16w+15 for Q K^T with its K fragments
// loaded straight from the pages (a B fragment is 16 contiguous bytes of a
// key row), the scores meet in a small LDS tile, every wave repeats the
// (cheap) softmax of the 16 rows, and wave w accumulates a quarter of the
// value columns of P V against V^T staged in LDS.  No K tile in LDS: three
// workgroups fit a CU at value sizes up to 256.  Key splits cover multiples
// of 64 keys; with nsplit > 1 unnormalised outputs and (max, sum) go to
// part_o [T, H, nsplit, dv] / part_ml [T, H, nsplit, 2] for the split merge.
template <int DKC, int DVT, bool VEC>
__global__ void __launch_bounds__(256) attn_heads_mfma_kernel(
    u16* __restrict__ out, const u16* __restrict__ q,
    const u16* __restrict__ kc, const u16* __restrict__ vc,
    const i32* __restrict__ bt, const i32* __restrict__ row_seq,
    const i32* __restrict__ positions, float scale, int H, int G, int dk,
    int dv, int page, int maxp, int chunk, int window, i64 ldq, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml, AttnExtra ex) {
  constexpr int VS = 72;             // V^T / P row stride (64 tokens + pad)
  constexpr int SS = 68;             // score row stride (floats)
  constexpr int DVW = DVT / 4;       // value tiles per wave
  __shared__ u16 v_lds[DVT * 16 * VS];
  __shared__ u16 p_lds[4 * 16 * VS];
  __shared__ float s_lds[16 * SS];
  __shared__ i32 row_lds[64];

  const int t = blockIdx.x, sp = blockIdx.z;
  const int hpg = H / G, nhb = (hpg + 15) / 16;
  const int g = blockIdx.y / nhb, hb = blockIdx.y % nhb;
  const int hbase = g * hpg + hb * 16;
  const int nrows = min(16, hpg - hb * 16);
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = positions[t];
  const i32* btr = bt + (size_t)row_seq[t] * maxp;
  int lo = 0, hi = pos;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0) lo = max(lo, pos - window + 1);
  // always-visible leading keys outside the window sit in front of it in a
  // virtual key index: [wlo - nf, wlo) stands for the keys [0, nf)
  const int wlo = lo;
  const int vsh = lo - (ex.first > 0 ? min(ex.first, lo) : 0);
  lo = vsh;
  if (nsplit > 1) {   // this workgroup's share of [lo, pos]; may be empty
    const int per = ((pos - lo + nsplit) / nsplit + 63) & ~63;
    lo += sp * per;
    hi = min(pos, lo + per - 1);
  }
  if (lo > hi && !(ex.sink && sp == 0)) {
    // an empty split (the grid is sized for the longest reach): mark it and
    // leave before touching queries or pages
    if ((int)threadIdx.x < nrows) {
      const size_t th = (size_t)t * H + hbase + threadIdx.x;
      part_ml[(th * nsplit + sp) * 2] = AF_NEG_INF;
      part_ml[(th * nsplit + sp) * 2 + 1] = 0.f;
    }
    return;
  }

  s16x8 q_frag[DKC];
  {
    const int head = hbase + min(lane & 15, nrows - 1);
    const u16* qr = q + (size_t)t * ldq + (size_t)head * dk;
#pragma unroll
    for (int c = 0; c < DKC; ++c)
      q_frag[c] = load8<VEC>(qr, c * 32 + (lane >> 4) * 8, dk);
  }
  float m[4], l[4], r1v[4], r2v[4];
  f32x4 o_acc[DVW];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int hr = (lane >> 4) * 4 + r;
    const int head = hbase + min(hr, nrows - 1);
    const bool sk = ex.sink && sp == 0 && hr < nrows;   // first split only
    m[r] = sk ? ex.sink[head] : AF_NEG_INF;
    l[r] = sk ? 1.f : 0.f;
    r1v[r] = ex.r1 ? ex.r1[head] : 0.f;
    r2v[r] = ex.r1 ? ex.r2[head] : 0.f;
  }
#pragma unroll
  for (int dw = 0; dw < DVW; ++dw) o_acc[dw] = f32x4{0.f, 0.f, 0.f, 0.f};
  u16* pw = p_lds + wid * 16 * VS;
  const float inv_cap = ex.cap > 0.f ? 1.0f / ex.cap : 0.f;

  for (int kv0 = lo; kv0 <= hi; kv0 += 64) {
    __syncthreads();   // the previous tile's scores, V^T and rows are read
    if (threadIdx.x < 64) {
      const int jv = kv0 + threadIdx.x;
      const int j = jv < wlo ? jv - vsh : jv;
      row_lds[threadIdx.x] =
          jv <= hi ? (btr[j / page] * G + g) * page + (j % page) : -1;
    }
    __syncthreads();
    // ---- this wave's 16 keys: K fragments from the pages ----
    s16x8 kf[DKC];
    {
      const int krow = row_lds[wid * 16 + (lane & 15)];
#pragma unroll
      for (int c = 0; c < DKC; ++c) {
        kf[c] = s16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (krow >= 0)
          kf[c] = load8<VEC>(kc + (size_t)krow * dk, c * 32 + (lane >> 4) * 8, dk);
      }
    }
    // ---- V^T of the whole tile, all threads ----
    constexpr int VIT = (32 * DVT * 2 + 255) / 256;
#pragma unroll
    for (int it = 0; it < VIT; ++it) {
      const int i = it * 256 + threadIdx.x;
      if (i >= 32 * DVT * 2) break;
      const int tp = i % 32, e0 = (i / 32) * 8;
      const int ra = row_lds[tp * 2], rb = row_lds[tp * 2 + 1];
      s16x8 a = {0, 0, 0, 0, 0, 0, 0, 0}, c8 = a;
      if (ra >= 0) a = load8<VEC>(vc + (size_t)ra * ex.ldv, e0, dv);
      if (rb >= 0) c8 = load8<VEC>(vc + (size_t)rb * ex.ldv, e0, dv);
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const uint32_t packed = (uint32_t)(unsigned short)a[jj] |
                                ((uint32_t)(unsigned short)c8[jj] << 16);
        *reinterpret_cast<uint32_t*>(v_lds + (e0 + jj) * VS + tp * 2) = packed;
      }
    }
    // ---- scores of the sub-tile, parked in C layout ----
    {
      f32x4 sa = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DKC; ++c)
        sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            as_bf16x8(q_frag[c]), as_bf16x8(kf[c]), sa, 0, 0, 0);
      const int jv = kv0 + wid * 16 + (lane & 15);
      const int j = jv < wlo ? jv - vsh : jv;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float sv = sa[r] * scale;
        if (ex.cap > 0.f) sv = attn_softcap_fast(sv, inv_cap, ex.cap);
        if (ex.r1) sv -= attn_dist_bias(r1v[r], r2v[r], max(pos - j, 0));
        s_lds[((lane >> 4) * 4 + r) * SS + wid * 16 + (lane & 15)] =
            (jv <= hi) ? sv : AF_NEG_INF;
      }
    }
    __syncthreads();
    // ---- softmax of the 16 rows over the tile, the same in every wave ----
    f32x4 s_acc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float sr[4];
      float tmax = AF_NEG_INF;
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        sr[st] = s_lds[((lane >> 4) * 4 + r) * SS + st * 16 + (lane & 15)];
        tmax = fmaxf(tmax, sr[st]);
      }
      tmax = group16_max_f32(tmax);
      const float mn = fmaxf(m[r], tmax);
      const float corr = (m[r] <= AF_NEG_INF) ? 0.f : __expf(m[r] - mn);
      float psum = 0.f;
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        sr[st] = (sr[st] <= AF_NEG_INF) ? 0.f : __expf(sr[st] - mn);
        psum += sr[st];
        s_acc[st][r] = sr[st];
      }
      l[r] = l[r] * corr + group16_sum_f32(psum);
      m[r] = mn;
#pragma unroll
      for (int dw = 0; dw < DVW; ++dw) o_acc[dw][r] *= corr;
    }
#pragma unroll
    for (int st = 0; st < 4; ++st)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        pw[((lane >> 4) * 4 + r) * VS + st * 16 + (lane & 15)] = f2bf(s_acc[st][r]);
    __builtin_amdgcn_wave_barrier();
    const s16x8 pf0 = *reinterpret_cast<const s16x8*>(pw + (lane & 15) * VS + (lane >> 4) * 8);
    const s16x8 pf1 = *reinterpret_cast<const s16x8*>(pw + (lane & 15) * VS + 32 + (lane >> 4) * 8);
    __builtin_amdgcn_wave_barrier();
    // ---- this wave's value columns ----
#pragma unroll
    for (int dw = 0; dw < DVW; ++dw) {
      const int dt = wid * DVW + dw;
      const u16* vrow = v_lds + (dt * 16 + (lane & 15)) * VS + (lane >> 4) * 8;
      const s16x8 vf0 = *reinterpret_cast<const s16x8*>(vrow);
      const s16x8 vf1 = *reinterpret_cast<const s16x8*>(vrow + 32);
      o_acc[dw] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          as_bf16x8(pf0), as_bf16x8(vf0), o_acc[dw], 0, 0, 0);
      o_acc[dw] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          as_bf16x8(pf1), as_bf16x8(vf1), o_acc[dw], 0, 0, 0);
    }
  }

#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int hr = (lane >> 4) * 4 + r;
    if (hr >= nrows) continue;
    const size_t th = (size_t)t * H + hbase + hr;
    if (nsplit == 1) {
      const float inv = l[r] > 0.f ? 1.0f / l[r] : 0.f;
#pragma unroll
      for (int dw = 0; dw < DVW; ++dw) {
        const int d = (wid * DVW + dw) * 16 + (lane & 15);
        if (d < dv) out[th * dv + d] = f2bf(o_acc[dw][r] * inv);
      }
    } else {
#pragma unroll
      for (int dw = 0; dw < DVW; ++dw) {
        const int d = (wid * DVW + dw) * 16 + (lane & 15);
        if (d < dv) part_o[(th * nsplit + sp) * dv + d] = o_acc[dw][r];
      }
      if (wid == 0 && (lane & 15) == 0) {
        part_ml[(th * nsplit + sp) * 2] = m[r];
        part_ml[(th * nsplit + sp) * 2 + 1] = l[r];
      }
    }
  }
}

}  // namespace

// q [T, H*dk] bf16 rows at stride ldq; caches [P, G, page, dk|dv] bf16;
// tile map (tile_seq, tile_q0): workgroup i covers chunk rows
// [q0, q0 + 64) of sequence tile_seq[i].  out [T, H*dv] bf16.
AF_EXPORT int afm_attn_prefill_mfma(
    void* out, const void* q, const void* kc, const void* vc, const void* bt,
    const void* cu, const void* q_start, const void* tile_seq,
    const void* tile_q0, float scale, int ntiles, int H, int G, int dk, int dv,
    int page, int maxp, int chunk, int window, i64 ldq, const void* sink,
    float cap, const void* r1, const void* r2, i64 ldv, int keep_first,
    void* stream) {
  if (ntiles == 0) return 0;
  if (keep_first < 0) return 9003;
  if (G <= 0 || H % G || dk < 1 || dv < 1) return 9003;
  if (ldv < dv || cap < 0.f || ((r1 == nullptr) != (r2 == nullptr))) return 9003;
  const bool vec = (dk % 8 == 0) && (dv % 8 == 0) && (ldq % 8 == 0) &&
                   (ldv % 8 == 0) &&
                   ((uintptr_t)q % 16 == 0) && ((uintptr_t)kc % 16 == 0) &&
                   ((uintptr_t)vc % 16 == 0);
  // wide heads exist in the 16-byte-aligned form only; 9004 sends the caller
  // to the row kernel
  if (dk > 576 || dv > 512 || ((dk > 128 || dv > 128) && !vec)) return 9004;
  const AttnExtra ex{(const float*)sink, (const float*)r1, (const float*)r2,
                     cap, ldv, keep_first};
  // two heads per workgroup when a K/V group has an even number of them
  const bool pair = vec && (H / G) % 2 == 0;
  hipStream_t s = (hipStream_t)stream;
#define APM(DKC, DVT, VEC, NH, ...)                                            \
  attn_prefill_mfma_kernel<DKC, DVT, VEC, NH, ##__VA_ARGS__>                   \
      <<<dim3(ntiles, H / NH), 256 * NH, 0, s>>>(                              \
      (u16*)out, (const u16*)q, (const u16*)kc, (const u16*)vc,                \
      (const i32*)bt, (const i32*)cu, (const i32*)q_start,                     \
      (const i32*)tile_seq, (const i32*)tile_q0, scale, H, G, dk, dv, page,    \
      maxp, chunk, window, ldq, ex)
  const bool small = dk <= 64 && dv <= 64;
  // the widest heads pair up over 32-key tiles: two heads' 64-key tiles are
  // 164 KB of LDS
  if (dk > 320 || dv > 256) {
    if (pair)
      attn_prefill_mfma_wide_pair_kernel<<<dim3(ntiles, H / 2), 512, 0, s>>>(
          (u16*)out, (const u16*)q, (const u16*)kc, (const u16*)vc,
          (const i32*)bt, (const i32*)cu, (const i32*)q_start,
          (const i32*)tile_seq, (const i32*)tile_q0, scale, H, G, dk, dv, page,
          maxp, chunk, window, ldq, ex);
    else
      APM(18, 32, true, 1);
  }
  else if (dk > 128 || dv > 128) { if (pair) APM(10, 16, true, 2); else APM(10, 16, true, 1); }
  else if (small && pair) APM(2, 4, true, 2);
  else if (small && vec) APM(2, 4, true, 1);
  else if (small) APM(2, 4, false, 1);
  else if (pair) APM(4, 8, true, 2);
  else if (vec) APM(4, 8, true, 1);
  else APM(4, 8, false, 1);
#undef APM
  return af_last_err();
}

// One row per token (decode steps): q [T, H*dk] at stride ldq, position and
// sequence of every row in positions / row_seq.  The caller merges the key
// splits (afm_attn_split_combine) when nsplit > 1.
AF_EXPORT int afm_attn_heads_mfma(
    void* out, const void* q, const void* kc, const void* vc, const void* bt,
    const void* row_seq, const void* positions, float scale, int T, int H,
    int G, int dk, int dv, int page, int maxp, int chunk, int window, i64 ldq,
    int nsplit, void* part_o, void* part_ml, const void* sink, float cap,
    const void* r1, const void* r2, i64 ldv, int keep_first, void* stream) {
  if (T == 0) return 0;
  if (keep_first < 0) return 9003;
  if (G <= 0 || H % G || dk < 1 || dv < 1) return 9003;
  if (ldv < dv || cap < 0.f || ((r1 == nullptr) != (r2 == nullptr))) return 9003;
  if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && (!part_o || !part_ml))) return 9003;
  const bool vec = (dk % 8 == 0) && (dv % 8 == 0) && (ldq % 8 == 0) &&
                   (ldv % 8 == 0) &&
                   ((uintptr_t)q % 16 == 0) && ((uintptr_t)kc % 16 == 0) &&
                   ((uintptr_t)vc % 16 == 0);
  if (dk > 576 || dv > 512 || ((dk > 128 || dv > 128) && !vec)) return 9004;
  const AttnExtra ex{(const float*)sink, (const float*)r1, (const float*)r2,
                     cap, ldv, keep_first};
  const int hpg = H / G;
  dim3 grid(T, G * ((hpg + 15) / 16), nsplit), blk(256);
  hipStream_t s = (hipStream_t)stream;
#define AHM(DKC, DVT, VEC)                                                     \
  attn_heads_mfma_kernel<DKC, DVT, VEC><<<grid, blk, 0, s>>>(                  \
      (u16*)out, (const u16*)q, (const u16*)kc, (const u16*)vc,                \
      (const i32*)bt, (const i32*)row_seq, (const i32*)positions, scale, H, G, \
      dk, dv, page, maxp, chunk, window, ldq, nsplit, (float*)part_o,          \
      (float*)part_ml, ex)
  const bool small = dk <= 64 && dv <= 64;
  if (dk > 320 || dv > 256) AHM(18, 32, true);
  else if (dk > 128 || dv > 128) AHM(10, 16, true);
  else if (small && vec) AHM(2, 4, true);
  else if (small) AHM(2, 4, false);
  else if (vec) AHM(4, 8, true);
  else AHM(4, 8, false);
#undef AHM
  return af_last_err();
}
