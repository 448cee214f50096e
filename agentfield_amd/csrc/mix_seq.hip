// Sequence mixers over packed row chunks: whole-row q/k RMSNorm + paged
// cache append, masked (causal / chunk-local / banded) paged softmax
// attention for arbitrary head sizes, and the token-serial decayed
// outer-product recurrence with per-sequence fp32 state slots.
//
// Storage dtype S is bf16 (raw u16) or fp32; scores, softmax, decays and the
// recurrent state are fp32.
#include "common.h"
#include "mix_attn.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// ---------------------------------------------------------------- qk norm
// One workgroup per row.  q row [nq], k row [nk], v row [nv]; caches
// [P, G, page, dk|dv]; slot = page_index*page + offset.  V = 4: 4-element
// vector accesses (sizes and strides multiples of 4), V = 1: scalar.
template <typename S, int V>
__device__ __forceinline__ void ldvs(const S* p, float (&o)[4]) {
  if (V == 4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = 0.f;
    if constexpr (sizeof(S) == 2) {
      const s16x4 v = *reinterpret_cast<const s16x4*>(p);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = bf2f((u16)v[j]);
    } else {
      const f32x4 v = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = v[j];
    }
  } else {
    o[0] = ldf<S>(p);
    o[1] = o[2] = o[3] = 0.f;
  }
}
template <typename S, int V>
__device__ __forceinline__ void stvs(S* p, const float (&o)[4]) {
  if (V == 4) {
    if constexpr (sizeof(S) == 2) {
      s16x4 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (short)f2bf(o[j]);
      *reinterpret_cast<s16x4*>(p) = v;
    } else {
      *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
    }
  } else {
    stf<S>(p, o[0]);
  }
}

template <typename S, int V>
__global__ void __launch_bounds__(256) qk_norm_cache_kernel(
    S* __restrict__ qout, const S* __restrict__ q, const S* __restrict__ k,
    const S* __restrict__ v, const S* __restrict__ qw, const S* __restrict__ kw,
    S* __restrict__ kc, S* __restrict__ vc, const i64* __restrict__ slots,
    float eps, int nq, int nk, int nv, int G, int dk, int dv, int page,
    i64 ldq, i64 ldk, i64 ldv) {
  __shared__ float red[8];
  const int t = blockIdx.x;
  const S* qr = q + (size_t)t * ldq;
  const S* kr = k + (size_t)t * ldk;
  const S* vr = v + (size_t)t * ldv;
  float sq = 0.f, sk = 0.f;
  float f[4], w4[4];
  for (int i = threadIdx.x * V; i < nq; i += 256 * V) {
    ldvs<S, V>(qr + i, f);
#pragma unroll
    for (int j = 0; j < V; ++j) sq += f[j] * f[j];
  }
  for (int i = threadIdx.x * V; i < nk; i += 256 * V) {
    ldvs<S, V>(kr + i, f);
#pragma unroll
    for (int j = 0; j < V; ++j) sk += f[j] * f[j];
  }
  sq = wave_sum_f32(sq);
  sk = wave_sum_f32(sk);
  if ((threadIdx.x & 63) == 0) {
    red[threadIdx.x >> 6] = sq;
    red[4 + (threadIdx.x >> 6)] = sk;
  }
  __syncthreads();
  const float rq = qw ? 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)nq + eps) : 1.0f;
  const float rk = kw ? 1.0f / sqrtf((red[4] + red[5] + red[6] + red[7]) / (float)nk + eps) : 1.0f;
  for (int i = threadIdx.x * V; i < nq; i += 256 * V) {
    ldvs<S, V>(qr + i, f);
    if (qw) {
      ldvs<S, V>(qw + i, w4);
#pragma unroll
      for (int j = 0; j < V; ++j) f[j] *= rq * w4[j];
    }
    stvs<S, V>(qout + (size_t)t * nq + i, f);
  }
  const i64 sl = slots[t];
  if (sl < 0) return;
  const i64 pg = sl / page, off = sl % page;
  for (int i = threadIdx.x * V; i < nk; i += 256 * V) {
    const int g = i / dk, d = i % dk;
    ldvs<S, V>(kr + i, f);
    if (kw) {
      ldvs<S, V>(kw + i, w4);
#pragma unroll
      for (int j = 0; j < V; ++j) f[j] *= rk * w4[j];
    }
    stvs<S, V>(kc + (((size_t)pg * G + g) * page + off) * dk + d, f);
  }
  for (int i = threadIdx.x * V; i < nv; i += 256 * V) {
    const int g = i / dv, d = i % dv;
    ldvs<S, V>(vr + i, f);
    stvs<S, V>(vc + (((size_t)pg * G + g) * page + off) * dv + d, f);
  }
}

// -------------------------------------------------------- masked attention
// One wave per (row, query head), 4 waves per workgroup.  Keys are walked in
// tiles of 64 (one key per lane for the scores, one output channel per lane
// for P.V), online softmax across tiles.  MAXV = ceil(dv/64) accumulators.
template <typename S, int MAXV>
__global__ void __launch_bounds__(256) masked_attention_kernel(
    S* __restrict__ out, const S* __restrict__ q, const S* __restrict__ kc,
    const S* __restrict__ vc, const i32* __restrict__ bt,
    const i32* __restrict__ row_seq, const i32* __restrict__ positions,
    float scale, int n_rh, int H, int G, int dk, int dv, int page, int maxp,
    int chunk, int window, i64 ldq, AttnExtra ex) {
  extern __shared__ float smem[];           // [4][dk + 64]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int rh = blockIdx.x * 4 + wave;
  if (rh >= n_rh) return;                    // whole wave exits together
  float* qs = smem + wave * (dk + 64);
  float* ps = qs + dk;
  const int t = rh / H, h = rh % H;
  const int g = h / (H / G);
  const int pos = positions[t];
  const i32* btr = bt + (size_t)row_seq[t] * maxp;
  int lo = 0;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
  // always-visible leading keys outside the window sit in front of it in a
  // virtual key index: [lo - nf, lo) stands for the keys [0, nf)
  const int nf = ex.first > 0 ? min(ex.first, lo) : 0;
  const int vsh = lo - nf;
  const S* qr = q + (size_t)t * ldq + (size_t)h * dk;
  for (int d = lane; d < dk; d += 64) qs[d] = ldf<S>(qr + d) * scale;
  float m = AF_NEG_INF, l = 0.f;
  if (ex.sink) { m = ex.sink[h]; l = 1.f; }
  const float r1 = ex.r1 ? ex.r1[h] : 0.f, r2 = ex.r1 ? ex.r2[h] : 0.f;
  float acc[MAXV];
#pragma unroll
  for (int i = 0; i < MAXV; ++i) acc[i] = 0.f;
  for (int j0 = vsh; j0 <= pos; j0 += 64) {
    const int jv = j0 + lane;
    const int j = jv < lo ? jv - vsh : jv;
    float s = AF_NEG_INF;
    if (jv <= pos) {
      const int pg = btr[j / page];
      const S* kr = kc + (((size_t)pg * G + g) * page + (j % page)) * dk;
      float d0 = 0.f;
      for (int d = 0; d < dk; ++d) d0 += qs[d] * ldf<S>(kr + d);
      s = attn_softcap(d0, ex.cap);
      if (ex.r1) s -= attn_dist_bias(r1, r2, pos - j);
    }
    const float mn = fmaxf(m, wave_max_f32(s));
    const float corr = (m <= AF_NEG_INF) ? 0.f : expf(m - mn);
    const float p = (jv <= pos) ? expf(s - mn) : 0.f;
    l = l * corr + wave_sum_f32(p);
    m = mn;
    __builtin_amdgcn_wave_barrier();
    ps[lane] = p;                            // wave-private LDS: ordered without a block barrier
    __builtin_amdgcn_wave_barrier();
    const int cnt = min(64, pos - j0 + 1);
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
      const int d = lane + 64 * i;
      float a = acc[i] * corr;
      if (d < dv) {
        for (int jj = 0; jj < cnt; ++jj) {
          const int jk = (j0 + jj) < lo ? j0 + jj - vsh : j0 + jj;
          const int pg = btr[jk / page];
          a += ps[jj] * ldf<S>(vc + (((size_t)pg * G + g) * page + (jk % page)) * ex.ldv + d);
        }
      }
      acc[i] = a;
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int d = lane + 64 * i;
    if (d < dv) stf<S>(out + ((size_t)t * H + h) * dv + d, acc[i] * inv);
  }
}

// ------------------------------------------------ row attention (decode)
// One workgroup per (row, K/V head): the GQ query heads of the group share
// every K and V load.  Keys are walked in super-tiles of `kt`:
//   A. scores: one key per lane, its row read 16 bytes at a time and dotted
//      with every head's query (queries sit in LDS, read as broadcasts), so
//      no cross-lane reduction is needed; one score per (head, key) in LDS;
//   B. per head: max, exp, sum over the tile (running max / sum / rescale
//      factor kept in LDS across super-tiles);
//   C. P.V: a value row is read by LPV adjacent lanes, each lane accumulates
//      its 16-byte slice for every head in registers.
// The partial outputs of the key groups are summed with shuffles, across
// waves through LDS.  Serves decode steps and short prompt portions, bf16
// and fp32 storage; head sizes up to 64 lanes x 16 bytes.
template <typename S, bool VEC>
__device__ __forceinline__ void load_slice(const S* row, int e0, int n,
                                           float (&o)[16 / sizeof(S)]) {
  constexpr int EPL = 16 / sizeof(S);
  if (VEC) {
    if (e0 < n) {
      if constexpr (sizeof(S) == 2) {
        const s16x8 v = *reinterpret_cast<const s16x8*>(row + e0);
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = bf2f((u16)v[j]);
      } else {
        const f32x4 v = *reinterpret_cast<const f32x4*>(row + e0);
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = v[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < EPL; ++j) o[j] = 0.f;
    }
  } else {
#pragma unroll
    for (int j = 0; j < EPL; ++j) o[j] = (e0 + j < n) ? ldf<S>(row + e0 + j) : 0.f;
  }
}

template <typename S, int GQ, bool VEC>
__global__ void __launch_bounds__(256) attn_rows_kernel(
    S* __restrict__ out, const S* __restrict__ q, const S* __restrict__ kc,
    const S* __restrict__ vc, const i32* __restrict__ bt,
    const i32* __restrict__ row_seq, const i32* __restrict__ positions,
    float scale, int H, int G, int dk, int dv, int page, int maxp, int chunk,
    int window, i64 ldq, int lpk_log2, int lpv_log2, int kt, int nsplit,
    float* __restrict__ part_o, float* __restrict__ part_ml, AttnExtra ex) {
  // nsplit > 1: the visible keys are cut into nsplit ranges, one workgroup
  // each (grid.z = head blocks x nsplit); unnormalised outputs and (max,
  // sum) go to part_o [T, H, nsplit, dv] / part_ml [T, H, nsplit, 2] and
  // attn_split_combine_kernel merges them.
  constexpr int EPL = 16 / sizeof(S);
  extern __shared__ float smem[];
  const int dvp = EPL << lpv_log2;             // padded value width
  float* sc = smem;                            // [GQ][kt] scores, then probabilities
  float* red = sc + GQ * kt;                   // [4][GQ][dvp]
  float* m_run = red + 4 * GQ * dvp;           // [8]
  float* l_run = m_run + 8;                    // [8]
  float* corr = l_run + 8;                     // [8]
  float* r1s = corr + 8;                       // [8] distance-bias factors
  float* r2s = r1s + 8;                        // [8]
  const int dkp = (dk + EPL - 1) / EPL * EPL;
  float* qs = r2s + 8;                         // [GQ][dkp] scaled queries
  const int t = blockIdx.x, g = blockIdx.y;
  const int hpg = H / G;
  const int zh = blockIdx.z / nsplit, sp = blockIdx.z % nsplit;
  const int h0 = g * hpg + zh * GQ;
  const int nh = min(GQ, hpg - zh * GQ);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int pos = positions[t];
  const int qpos = pos;
  const i32* btr = bt + (size_t)row_seq[t] * maxp;
  int lo = 0;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0 && pos - window + 1 > lo) lo = pos - window + 1;
  // always-visible leading keys outside the window sit in front of it in a
  // virtual key index: [wlo - nf, wlo) stands for the keys [0, nf)
  const int wlo = lo;
  const int vsh = lo - (ex.first > 0 ? min(ex.first, lo) : 0);
  lo = vsh;
  if (nsplit > 1) {   // this workgroup's share of [lo, pos]; may be empty
    const int per = (pos - lo + nsplit) / nsplit;
    lo += sp * per;
    pos = min(pos, lo + per - 1);
  }

  const int liv = lane & ((1 << lpv_log2) - 1), kiv = lane >> lpv_log2;
  const int kpv = 64 >> lpv_log2;

  for (int i = threadIdx.x; i < GQ * dkp; i += 256) {
    const int gg = i / dkp, d = i % dkp;
    qs[i] = (gg < nh && d < dk)
        ? ldf<S>(q + (size_t)t * ldq + (size_t)(h0 + gg) * dk + d) * scale : 0.f;
  }
  float acc[GQ][EPL];
#pragma unroll
  for (int gg = 0; gg < GQ; ++gg)
#pragma unroll
    for (int j = 0; j < EPL; ++j) acc[gg][j] = 0.f;
  if (threadIdx.x < GQ) {
    // the sink joins the first key range only
    const bool sk = ex.sink && sp == 0 && (int)threadIdx.x < nh;
    m_run[threadIdx.x] = sk ? ex.sink[h0 + threadIdx.x] : AF_NEG_INF;
    l_run[threadIdx.x] = sk ? 1.f : 0.f;
    const bool rb = ex.r1 && (int)threadIdx.x < nh;
    r1s[threadIdx.x] = rb ? ex.r1[h0 + threadIdx.x] : 0.f;
    r2s[threadIdx.x] = rb ? ex.r2[h0 + threadIdx.x] : 0.f;
  }

  for (int tile0 = lo; tile0 <= pos; tile0 += kt) {
    const int nk = min(kt, pos + 1 - tile0);
    // ---- A: scores, one key per lane ----
    if (tile0 == lo) __syncthreads();          // queries are in LDS
    for (int kidx = threadIdx.x; kidx < nk; kidx += 256) {
      const int jv = tile0 + kidx;
      const int j = jv < wlo ? jv - vsh : jv;
      const S* kr = kc + (((size_t)btr[j / page] * G + g) * page + (j % page)) * dk;
      float sco[GQ];
#pragma unroll
      for (int gg = 0; gg < GQ; ++gg) sco[gg] = 0.f;
#pragma unroll 4
      for (int e0 = 0; e0 < dk; e0 += EPL) {
        float kv[EPL];
        load_slice<S, VEC>(kr, e0, dk, kv);
#pragma unroll
        for (int gg = 0; gg < GQ; ++gg)
#pragma unroll
          for (int e = 0; e < EPL; ++e) sco[gg] += qs[gg * dkp + e0 + e] * kv[e];
      }
#pragma unroll
      for (int gg = 0; gg < GQ; ++gg)
        if (gg < nh) {
          float sv = attn_softcap(sco[gg], ex.cap);
          if (ex.r1) sv -= attn_dist_bias(r1s[gg], r2s[gg], qpos - j);
          sc[gg * kt + kidx] = sv;
        }
    }
    __syncthreads();
    // ---- B: softmax statistics, wave w takes heads w, w+4, ... ----
    for (int gg = wave; gg < nh; gg += 4) {
      float* sr = sc + gg * kt;
      float mx = AF_NEG_INF;
      for (int i = lane; i < nk; i += 64) mx = fmaxf(mx, sr[i]);
      mx = wave_max_f32(mx);
      const float m_old = m_run[gg];
      const float m_new = fmaxf(m_old, mx);
      float sum = 0.f;
      for (int i = lane; i < nk; i += 64) {
        const float p = expf(sr[i] - m_new);
        sr[i] = p;
        sum += p;
      }
      sum = wave_sum_f32(sum);
      if (lane == 0) {
        const float c = (m_old <= AF_NEG_INF) ? 0.f : expf(m_old - m_new);
        corr[gg] = c;
        l_run[gg] = l_run[gg] * c + sum;
        m_run[gg] = m_new;
      }
    }
    __syncthreads();
    // ---- C: accumulate P.V ----
    if (tile0 > lo) {
#pragma unroll
      for (int gg = 0; gg < GQ; ++gg) {
        const float c = gg < nh ? corr[gg] : 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[gg][e] *= c;
      }
    }
    for (int kb = wave * kpv; kb < nk; kb += 16 * kpv) {
      float vv[4][EPL];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int jv = tile0 + min(kb + u * 4 * kpv + kiv, nk - 1);
        const int j = jv < wlo ? jv - vsh : jv;
        const S* vr = vc + (((size_t)btr[j / page] * G + g) * page + (j % page)) * ex.ldv;
        load_slice<S, VEC>(vr, liv * EPL, dv, vv[u]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int kidx = kb + u * 4 * kpv + kiv;
        const bool valid = kidx < nk;
#pragma unroll
        for (int gg = 0; gg < GQ; ++gg) {
          const float p = (valid && gg < nh) ? sc[gg * kt + kidx] : 0.f;
#pragma unroll
          for (int e = 0; e < EPL; ++e) acc[gg][e] += p * vv[u][e];
        }
      }
    }
    __syncthreads();   // scores of this tile are dead; next tile may overwrite
  }
  // ---- sum the key groups of a wave, then the 4 waves ----
#pragma unroll
  for (int gg = 0; gg < GQ; ++gg)
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
      float a = acc[gg][e];
      for (int o = 1 << lpv_log2; o < 64; o <<= 1) a += __shfl_xor(a, o, 64);
      if (kiv == 0) red[(wave * GQ + gg) * dvp + liv * EPL + e] = a;
    }
  __syncthreads();
  for (int i = threadIdx.x; i < nh * dv; i += 256) {
    const int gg = i / dv, d = i % dv;
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) o += red[(w * GQ + gg) * dvp + d];
    if (nsplit == 1)
      stf<S>(out + ((size_t)t * H + h0 + gg) * dv + d, o / l_run[gg]);
    else
      part_o[(((size_t)t * H + h0 + gg) * nsplit + sp) * dv + d] = o;
  }
  if (nsplit > 1 && threadIdx.x < nh) {
    float* ml = part_ml + (((size_t)t * H + h0 + threadIdx.x) * nsplit + sp) * 2;
    ml[0] = m_run[threadIdx.x];
    ml[1] = l_run[threadIdx.x];
  }
}

// One wave per (row, head): merge the nsplit (<= 64) partial softmaxes.
// Lane s weighs split s once; empty splits (max = -inf) weigh nothing and
// their partial outputs are never read.
template <typename S>
__global__ void __launch_bounds__(256) attn_split_combine_kernel(
    S* __restrict__ out, const float* __restrict__ part_o,
    const float* __restrict__ part_ml, int n_rh, int nsplit, int dv) {
  const int rh = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (rh >= n_rh) return;
  const int lane = threadIdx.x & 63;
  const float* ml = part_ml + (size_t)rh * nsplit * 2;
  const float ms = lane < nsplit ? ml[2 * lane] : AF_NEG_INF;
  const float ls = lane < nsplit ? ml[2 * lane + 1] : 0.f;
  const float m = wave_max_f32(ms);
  const float w = ms > AF_NEG_INF ? expf(ms - m) : 0.f;
  const float inv = 1.0f / wave_sum_f32(w * ls);
  for (int d0 = 0; d0 < dv; d0 += 64) {
    const int d = d0 + lane;
    float o = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float ws = __shfl(w, s, 64);
      if (ws > 0.f && d < dv)
        o += part_o[((size_t)rh * nsplit + s) * dv + d] * ws;
    }
    if (d < dv) stf<S>(out + (size_t)rh * dv + d, o * inv);
  }
}

// ------------------------------------------------------------- linear scan
// Workgroup = (sequence, head, 32-column tile of dv); 256 threads = 16 row
// groups x 16 column pairs.  Thread (r, c) keeps RP consecutive rows
// r*RP .. r*RP+RP-1 of columns c and c+16 of the state in registers (each
// q / k / decay value read from LDS feeds two columns).  Tokens are
// walked serially in blocks of TB: the block's q / k / decay rows are staged
// into LDS at once (rotary + scaling applied on the way in), every thread
// then advances its rows through the TB tokens without synchronising and
// leaves one partial output per token in LDS, and the 16 partials of each
// (token, column) are summed after one more barrier: two barriers per TB
// tokens, the recurrence itself strictly token by token in fp32 — so results
// are bit-identical however a sequence is cut into chunks.
template <typename S, int RP>
__global__ void __launch_bounds__(256) linear_scan_kernel(
    float* __restrict__ out, float* __restrict__ state,
    const S* __restrict__ q, const S* __restrict__ k, const S* __restrict__ v,
    const S* __restrict__ zl, const float* __restrict__ zbias,
    const float* __restrict__ head_decay, const float* __restrict__ inv_freq,
    const i32* __restrict__ positions, const i32* __restrict__ cu,
    const i32* __restrict__ q_start, const i32* __restrict__ sslot,
    float q_scale, float k_scale, float inv_tau, int H, int dk, int dv,
    int rot, i64 ldq, i64 ldk, i64 ldv, i64 ldz) {
  constexpr int DKP = 16 * RP;         // padded rows: zeros beyond dk
  // bf16 operands carry 2^-9 relative rounding already: hardware
  // transcendentals there; fp32 storage keeps the precise library forms
  constexpr bool FAST = sizeof(S) == 2;
  constexpr int SCAN_TB = RP >= 16 ? 8 : 16;  // keeps LDS under 64 KB
  extern __shared__ float smem[];      // [TB][3][DKP] + [TB][16][32] + [TB][32]
  const int b = blockIdx.x, h = blockIdx.y, c0 = blockIdx.z * 32;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t1 <= t0) return;
  const int r = threadIdx.x >> 4, cc = threadIdx.x & 15;
  const int ca = c0 + cc, cb = c0 + cc + 16;
  const bool oka = ca < dv, okb = cb < dv;
  float* stage = smem;                         // [TB][3][DKP]: q, k, decay
  float* part = smem + SCAN_TB * 3 * DKP;      // [TB][16][32]
  float* vs = part + SCAN_TB * 512;            // [TB][32]
  float* sbase = state + (((size_t)sslot[b] * H + h) * dk) * dv;
  float sta[RP], stb[RP];
  const bool fresh = q_start[b] == 0;
#pragma unroll
  for (int ii = 0; ii < RP; ++ii) {
    const int i = r * RP + ii;
    sta[ii] = (!fresh && oka && i < dk) ? sbase[(size_t)i * dv + ca] : 0.f;
    stb[ii] = (!fresh && okb && i < dk) ? sbase[(size_t)i * dv + cb] : 0.f;
  }
  const float hd = head_decay ? head_decay[h] : 1.0f;
  const int half = rot >> 1;
  // raw operands of the next block, fetched while the current one computes
  constexpr int EPT = SCAN_TB * DKP / 256;   // staged elements per thread
  float rq[EPT], rk[EPT], rqp[EPT], rkp[EPT], rz[EPT], rpos[EPT];
  float rv[(SCAN_TB * 32 + 255) / 256];
  // Every load is unconditional on a clamped address (invalid lanes are
  // zeroed afterwards), so all of a block's loads are in flight together
  // instead of one exposed memory latency per guarded element.
  auto fetch = [&](int tb) {
    const int nt = min(SCAN_TB, t1 - tb);
#pragma unroll
    for (int n = 0; n < EPT; ++n) {
      const int e = threadIdx.x + 256 * n;
      const int tt = e / DKP, i = e % DKP;
      const bool valid = tt < nt && i < dk;
      const int t = tb + min(tt, nt - 1), ic = min(i, dk - 1);
      const float a = ldf<S>(q + (size_t)t * ldq + (size_t)h * dk + ic);
      const float c = ldf<S>(k + (size_t)t * ldk + (size_t)h * dk + ic);
      rq[n] = valid ? a : 0.f;
      rk[n] = valid ? c : 0.f;
      rqp[n] = rkp[n] = rz[n] = rpos[n] = 0.f;
    }
    if (rot > 0) {
#pragma unroll
      for (int n = 0; n < EPT; ++n) {
        const int e = threadIdx.x + 256 * n;
        const int tt = e / DKP, i = e % DKP;
        const int t = tb + min(tt, nt - 1), ic = min(i, dk - 1);
        const int pi = ic < half ? ic + half : (ic < rot ? ic - half : ic);
        rqp[n] = ldf<S>(q + (size_t)t * ldq + (size_t)h * dk + pi);
        rkp[n] = ldf<S>(k + (size_t)t * ldk + (size_t)h * dk + pi);
        rpos[n] = (float)positions[t];
      }
    }
    if (zl) {
#pragma unroll
      for (int n = 0; n < EPT; ++n) {
        const int e = threadIdx.x + 256 * n;
        const int tt = e / DKP, i = e % DKP;
        const int t = tb + min(tt, nt - 1), ic = min(i, dk - 1);
        rz[n] = ldf<S>(zl + (size_t)t * ldz + (size_t)h * dk + ic);
      }
    }
#pragma unroll
    for (int n = 0; n < (SCAN_TB * 32 + 255) / 256; ++n) {
      const int e = threadIdx.x + 256 * n;
      const int tt = e >> 5, ci = c0 + (e & 31);
      const float x = ldf<S>(v + (size_t)(tb + min(tt, nt - 1)) * ldv +
                             (size_t)h * dv + min(ci, dv - 1));
      rv[n] = (tt < nt && ci < dv) ? x : 0.f;
    }
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += SCAN_TB) {
    const int nt = min(SCAN_TB, t1 - tb);
    // ---- stage the block: rotate / scale q, k; evaluate the decays ----
#pragma unroll
    for (int n = 0; n < EPT; ++n) {
      const int e = threadIdx.x + 256 * n;
      const int tt = e / DKP, i = e % DKP;
      float* row = stage + (size_t)tt * 3 * DKP;
      float qv = rq[n], kv = rk[n], a = 0.f;
      if (tt < nt && i < dk) {
        if (i < rot) {
          const bool lowh = i < half;
          float sn, cs;
          const float ang = rpos[n] * inv_freq[lowh ? i : i - half];
          if (FAST) { sn = __sinf(ang); cs = __cosf(ang); }
          else sincosf(ang, &sn, &cs);
          // pair (u, w) -> (u cos - w sin, w cos + u sin)
          qv = lowh ? qv * cs - rqp[n] * sn : qv * cs + rqp[n] * sn;
          kv = lowh ? kv * cs - rkp[n] * sn : kv * cs + rkp[n] * sn;
        }
        qv *= q_scale;
        kv *= k_scale;
        a = hd;
        if (zl) {
          const float z = rz[n] + zbias[(size_t)h * dk + i];
          // log(sigmoid(z)) = -softplus(-z), evaluated without overflow
          if (FAST) {
            const float ls = z >= 0.f ? -__logf(1.0f + __expf(-z))
                                      : z - __logf(1.0f + __expf(z));
            a = __expf(ls * inv_tau);
          } else {
            const float ls = z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
            a = expf(ls * inv_tau);
          }
        }
      }
      if (tt < SCAN_TB) {
        row[i] = qv;
        row[DKP + i] = kv;
        row[2 * DKP + i] = a;
      }
    }
#pragma unroll
    for (int n = 0; n < (SCAN_TB * 32 + 255) / 256; ++n) {
      const int e = threadIdx.x + 256 * n;
      if (e < SCAN_TB * 32) vs[e] = rv[n];
    }
    __syncthreads();
    if (tb + SCAN_TB < t1) fetch(tb + SCAN_TB);   // in flight during compute
    // ---- advance this thread's rows through the block, token by token ----
    auto step = [&](int tt) {
      const f32x2* sq = reinterpret_cast<const f32x2*>(
          stage + (size_t)tt * 3 * DKP + r * RP);
      const f32x2* sk = sq + DKP / 2;
      const f32x2* sa = sk + DKP / 2;
      const float va = vs[tt * 32 + cc], vb = vs[tt * 32 + cc + 16];
      float pa = 0.f, pb = 0.f;
#pragma unroll
      for (int i2 = 0; i2 < RP / 2; ++i2) {
        const f32x2 a2 = sa[i2], k2 = sk[i2], q2 = sq[i2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int ii = i2 * 2 + j;
          sta[ii] = a2[j] * sta[ii] + k2[j] * va;
          stb[ii] = a2[j] * stb[ii] + k2[j] * vb;
          pa += sta[ii] * q2[j];
          pb += stb[ii] * q2[j];
        }
      }
      part[tt * 512 + r * 32 + cc] = pa;
      part[tt * 512 + r * 32 + cc + 16] = pb;
    };
    if (nt == SCAN_TB) {
      // full block: fixed trip count, so the LDS reads of later tokens are
      // scheduled under the arithmetic of earlier ones
#pragma unroll
      for (int tt = 0; tt < SCAN_TB; ++tt) step(tt);
    } else {
      for (int tt = 0; tt < nt; ++tt) step(tt);
    }
    __syncthreads();
    // ---- o[t][c] = sum of the 16 row-group partials ----
    for (int e = threadIdx.x; e < nt * 32; e += 256) {
      const int tt = e >> 5, ci = e & 31;
      if (c0 + ci < dv) {
        const float* pr = part + tt * 512 + ci;
        float o = 0.f;
#pragma unroll
        for (int rr = 0; rr < 16; ++rr) o += pr[rr * 32];
        out[(size_t)(tb + tt) * H * dv + (size_t)h * dv + c0 + ci] = o;
      }
    }
    // the next block's staging writes `stage`/`vs`, last read before the
    // barrier above; its partials are written after the next barrier
  }
#pragma unroll
  for (int ii = 0; ii < RP; ++ii) {
    const int i = r * RP + ii;
    if (i < dk && oka) sbase[(size_t)i * dv + ca] = sta[ii];
    if (i < dk && okb) sbase[(size_t)i * dv + cb] = stb[ii];
  }
}

}  // namespace

AF_EXPORT int afm_qk_norm_cache(
    void* qout, const void* q, const void* k, const void* v, const void* qw,
    const void* kw, void* kc, void* vc, const void* slots, float eps, int T,
    int nq, int nk, int nv, int G, int dk, int dv, int page, i64 ldq, i64 ldk,
    i64 ldv, int dt, void* stream) {
  if (T == 0) return 0;
  if (nk != G * dk || nv != G * dv) return 9003;
  hipStream_t s = (hipStream_t)stream;
  auto al = [](const void* p) { return p == nullptr || (uintptr_t)p % 16 == 0; };
  const bool vec = dk % 4 == 0 && dv % 4 == 0 && nq % 4 == 0 && ldq % 4 == 0 &&
                   ldk % 4 == 0 && ldv % 4 == 0 && al(qout) && al(q) && al(k) &&
                   al(v) && al(qw) && al(kw) && al(kc) && al(vc);
#define QKN(ST, V)                                                            \
  qk_norm_cache_kernel<ST, V><<<T, 256, 0, s>>>((ST*)qout, (const ST*)q,      \
      (const ST*)k, (const ST*)v, (const ST*)qw, (const ST*)kw, (ST*)kc,      \
      (ST*)vc, (const i64*)slots, eps, nq, nk, nv, G, dk, dv, page, ldq, ldk, \
      ldv)
  if (dt == 0) { if (vec) QKN(u16, 4); else QKN(u16, 1); }
  else if (dt == 1) { if (vec) QKN(float, 4); else QKN(float, 1); }
  else return 9002;
#undef QKN
  return af_last_err();
}

template <typename S>
static int launch_attention(void* out, const void* q, const void* kc,
                            const void* vc, const void* bt, const void* row_seq,
                            const void* positions, float scale, int T, int H,
                            int G, int dk, int dv, int page, int maxp,
                            int chunk, int window, i64 ldq, int nsplit,
                            float* part_o, float* part_ml, AttnExtra ex,
                            hipStream_t s) {
  constexpr int EPL = 16 / (int)sizeof(S);
  if (dk <= 64 * EPL && dv <= 64 * EPL) {
    auto clog2 = [](int n) { int l = 0; while ((1 << l) < n) ++l; return l; };
    const int lpk = clog2((dk + EPL - 1) / EPL), lpv = clog2((dv + EPL - 1) / EPL);
    const int hpg = H / G;
    const int gq = hpg >= 8 ? 8 : hpg > 2 ? 4 : hpg;   // 1, 2, 4 or 8
    const int dvp = EPL << lpv;
    const int kt = dvp <= 128 ? 1024 : 512;
    const int dkp = (dk + EPL - 1) / EPL * EPL;
    const size_t sm = ((size_t)gq * kt + 4 * gq * dvp + 40 +
                       (size_t)gq * dkp) * sizeof(float);
    const bool vec = dk % EPL == 0 && dv % EPL == 0 && ex.ldv % EPL == 0 &&
                     (uintptr_t)kc % 16 == 0 && (uintptr_t)vc % 16 == 0;
    if (nsplit < 1 || nsplit > 64 || (nsplit > 1 && (!part_o || !part_ml))) return 9003;
    dim3 grid(T, G, ((hpg + gq - 1) / gq) * nsplit);
#define ROWS(GQ, VEC)                                                         \
  attn_rows_kernel<S, GQ, VEC><<<grid, 256, sm, s>>>(                         \
      (S*)out, (const S*)q, (const S*)kc, (const S*)vc, (const i32*)bt,       \
      (const i32*)row_seq, (const i32*)positions, scale, H, G, dk, dv, page,  \
      maxp, chunk, window, ldq, lpk, lpv, kt, nsplit, part_o, part_ml, ex)
    if (vec) {
      if (gq == 1) ROWS(1, true); else if (gq == 2) ROWS(2, true);
      else if (gq == 4) ROWS(4, true); else ROWS(8, true);
    } else {
      if (gq == 1) ROWS(1, false); else if (gq == 2) ROWS(2, false);
      else if (gq == 4) ROWS(4, false); else ROWS(8, false);
    }
#undef ROWS
    if (nsplit > 1)
      attn_split_combine_kernel<S><<<(T * H + 3) / 4, 256, 0, s>>>(
          (S*)out, part_o, part_ml, T * H, nsplit, dv);
    return af_last_err();
  }
  // very wide heads: one wave per (row, head), scalar key walk
  const int n_rh = T * H;
  const int grid = (n_rh + 3) / 4;
  const size_t sm = (size_t)4 * (dk + 64) * sizeof(float);
#define ATT(MV)                                                              \
  masked_attention_kernel<S, MV><<<grid, 256, sm, s>>>(                      \
      (S*)out, (const S*)q, (const S*)kc, (const S*)vc, (const i32*)bt,      \
      (const i32*)row_seq, (const i32*)positions, scale, n_rh, H, G, dk, dv, \
      page, maxp, chunk, window, ldq, ex)
  if (dv <= 64) ATT(1);
  else if (dv <= 128) ATT(2);
  else if (dv <= 256) ATT(4);
  else if (dv <= 512) ATT(8);
  else ATT(16);
#undef ATT
  return af_last_err();
}

AF_EXPORT int afm_masked_attention(
    void* out, const void* q, const void* kc, const void* vc, const void* bt,
    const void* row_seq, const void* positions, float scale, int T, int H,
    int G, int dk, int dv, int page, int maxp, int chunk, int window, i64 ldq,
    int nsplit, void* part_o, void* part_ml, const void* sink, float cap,
    const void* r1, const void* r2, i64 ldv, int keep_first, int dt,
    void* stream) {
  if (T == 0) return 0;
  if (G <= 0 || H % G || dv > 1024 || dk > 2048) return 9003;
  if (ldv < dv || cap < 0.f || ((r1 == nullptr) != (r2 == nullptr))) return 9003;
  if (keep_first < 0) return 9003;
  const AttnExtra ex{(const float*)sink, (const float*)r1, (const float*)r2,
                     cap, ldv, keep_first};
  hipStream_t s = (hipStream_t)stream;
  if (dt == 0)
    return launch_attention<u16>(out, q, kc, vc, bt, row_seq, positions, scale,
                                 T, H, G, dk, dv, page, maxp, chunk, window,
                                 ldq, nsplit, (float*)part_o, (float*)part_ml,
                                 ex, s);
  if (dt == 1)
    return launch_attention<float>(out, q, kc, vc, bt, row_seq, positions,
                                   scale, T, H, G, dk, dv, page, maxp, chunk,
                                   window, ldq, nsplit, (float*)part_o,
                                   (float*)part_ml, ex, s);
  return 9002;
}

// out [T*H, dv] bf16 from part_o [T*H, nsplit, dv] / part_ml [T*H, nsplit, 2].
AF_EXPORT int afm_attn_split_combine(void* out, const void* part_o,
                                     const void* part_ml, int n_rh, int nsplit,
                                     int dv, int dt, void* stream) {
  if (n_rh == 0) return 0;
  if (nsplit < 1 || nsplit > 64) return 9003;
  hipStream_t s = (hipStream_t)stream;
  if (dt == 0)
    attn_split_combine_kernel<u16><<<(n_rh + 3) / 4, 256, 0, s>>>(
        (u16*)out, (const float*)part_o, (const float*)part_ml, n_rh, nsplit, dv);
  else if (dt == 1)
    attn_split_combine_kernel<float><<<(n_rh + 3) / 4, 256, 0, s>>>(
        (float*)out, (const float*)part_o, (const float*)part_ml, n_rh, nsplit, dv);
  else
    return 9002;
  return af_last_err();
}

template <typename S>
static int launch_scan(float* out, float* state, const void* q, const void* k,
                       const void* v, const void* zl, const float* zbias,
                       const float* head_decay, const float* inv_freq,
                       const i32* positions, const i32* cu, const i32* q_start,
                       const i32* sslot, float q_scale, float k_scale,
                       float inv_tau, int B, int H, int dk, int dv, int rot,
                       i64 ldq, i64 ldk, i64 ldv, i64 ldz, hipStream_t s) {
  dim3 grid(B, H, (dv + 31) / 32);
  const int rp = (dk + 15) / 16;
  const int rpp = rp <= 2 ? 2 : rp <= 4 ? 4 : rp <= 8 ? 8 : 16;
  const size_t sm = (size_t)(rpp >= 16 ? 8 : 16) * (3 * 16 * rpp + 512 + 32) * sizeof(float);
#define SCAN(RP)                                                             \
  linear_scan_kernel<S, RP><<<grid, 256, sm, s>>>(                           \
      out, state, (const S*)q, (const S*)k, (const S*)v, (const S*)zl, zbias, \
      head_decay, inv_freq, positions, cu, q_start, sslot, q_scale, k_scale, \
      inv_tau, H, dk, dv, rot, ldq, ldk, ldv, ldz)
  if (rp <= 2) SCAN(2);
  else if (rp <= 4) SCAN(4);
  else if (rp <= 8) SCAN(8);
  else SCAN(16);
#undef SCAN
  return af_last_err();
}

AF_EXPORT int afm_linear_scan(
    void* out, void* state, const void* q, const void* k, const void* v,
    const void* zl, const void* zbias, const void* head_decay,
    const void* inv_freq, const void* positions, const void* cu,
    const void* q_start, const void* sslot, float q_scale, float k_scale,
    float inv_tau, int B, int H, int dk, int dv, int rot, i64 ldq, i64 ldk,
    i64 ldv, i64 ldz, int dt, void* stream) {
  if (B == 0) return 0;
  if (dk > 256 || dk < 1 || dv < 1) return 9003;
  if (rot < 0 || rot > dk || (rot & 1) || (rot && !inv_freq)) return 9003;
  if ((zl == nullptr) == (head_decay == nullptr)) return 9003;
  if (zl && !zbias) return 9003;
  hipStream_t s = (hipStream_t)stream;
  if (dt == 0)
    return launch_scan<u16>((float*)out, (float*)state, q, k, v, zl,
        (const float*)zbias, (const float*)head_decay, (const float*)inv_freq,
        (const i32*)positions, (const i32*)cu, (const i32*)q_start,
        (const i32*)sslot, q_scale, k_scale, inv_tau, B, H, dk, dv, rot, ldq,
        ldk, ldv, ldz, s);
  if (dt == 1)
    return launch_scan<float>((float*)out, (float*)state, q, k, v, zl,
        (const float*)zbias, (const float*)head_decay, (const float*)inv_freq,
        (const i32*)positions, (const i32*)cu, (const i32*)q_start,
        (const i32*)sslot, q_scale, k_scale, inv_tau, B, H, dk, dv, rot, ldq,
        ldk, ldv, ldz, s);
  return 9002;
}
