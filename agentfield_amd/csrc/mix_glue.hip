// Row-wise glue kernels of parallel-residual hybrid decoders: fp32 residual
// stream, zero-centred RMSNorm pairs with token shift, per-head output norm
// with SiLU gate, PolyNorm activation, sigmoid-gated residual add, softcap.
//
// Storage dtype S is bf16 (raw u16) or fp32; every statistic, gate and the
// residual itself are fp32.  One workgroup (256 threads = 4 waves) per row
// unless noted; rows are short (model width), so a row is read once into
// registers/LDS-free strided loops and reduced with 64-wide wave shuffles.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// 4 consecutive elements (8 B of bf16 / 16 B of fp32); callers guarantee the
// alignment (row lengths and strides multiples of 4, 16-byte aligned bases).
template <typename S> __device__ __forceinline__ void ld4(const S* p, float (&o)[4]);
template <> __device__ __forceinline__ void ld4<u16>(const u16* p, float (&o)[4]) {
  const s16x4 v = *reinterpret_cast<const s16x4*>(p);
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = bf2f((u16)v[j]);
}
template <> __device__ __forceinline__ void ld4<float>(const float* p, float (&o)[4]) {
  const f32x4 v = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = v[j];
}
template <typename S> __device__ __forceinline__ void st4(S* p, const float (&o)[4]);
template <> __device__ __forceinline__ void st4<u16>(u16* p, const float (&o)[4]) {
  s16x4 v;
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = (short)f2bf(o[j]);
  *reinterpret_cast<s16x4*>(p) = v;
}
template <> __device__ __forceinline__ void st4<float>(float* p, const float (&o)[4]) {
  *reinterpret_cast<f32x4*>(p) = f32x4{o[0], o[1], o[2], o[3]};
}
// V = 4: vector accesses; V = 1: scalar fallback for odd sizes.
template <typename S, int V>
__device__ __forceinline__ void ldv(const S* p, float (&o)[4]) {
  if (V == 4) ld4<S>(p, o);
  else { o[0] = ldf<S>(p); o[1] = o[2] = o[3] = 0.f; }
}
template <typename S, int V>
__device__ __forceinline__ void stv(S* p, const float (&o)[4]) {
  if (V == 4) st4<S>(p, o);
  else stf<S>(p, o[0]);
}

// Block-wide sum of up to N values per thread (256 threads); every thread
// gets the totals.  red must hold N*4 floats.
template <int N>
__device__ __forceinline__ void block_sum(float (&v)[N], float* red) {
#pragma unroll
  for (int n = 0; n < N; ++n) v[n] = wave_sum_f32(v[n]);
  const int wave = threadIdx.x >> 6;
  __syncthreads();  // red may still be read from a previous call
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int n = 0; n < N; ++n) red[n * 4 + wave] = v[n];
  }
  __syncthreads();
#pragma unroll
  for (int n = 0; n < N; ++n)
    v[n] = red[n * 4] + red[n * 4 + 1] + red[n * 4 + 2] + red[n * 4 + 3];
}

template <typename S>
__global__ void __launch_bounds__(256) embed_kernel(
    float* __restrict__ out, const S* __restrict__ table,
    const i32* __restrict__ ids, const float* __restrict__ add, float scale,
    int W) {
  const int t = blockIdx.x;
  const S* src = table + (size_t)ids[t] * W;
  float* dst = out + (size_t)t * W;
  for (int i = threadIdx.x; i < W; i += 256)
    dst[i] = ldf<S>(src + i) * scale + (add ? add[i] : 0.f);
}

__global__ void __launch_bounds__(256) add_rows_kernel(
    float* __restrict__ x, const float* __restrict__ other,
    const float* __restrict__ vec, i64 n, int W) {
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    float v = x[i];
    if (other) v += other[i];
    if (vec) v += vec[i % W];
    x[i] = v;
  }
}

// a = norm(x)(1+w1), b = norm(x)(1+w2), s = a + (a_prev - a)*shift.
template <typename S, int V>
__global__ void __launch_bounds__(256) dual_norm_shift_kernel(
    S* __restrict__ a_out, S* __restrict__ s_out, S* __restrict__ b_out,
    float* __restrict__ last, const float* __restrict__ x,
    const S* __restrict__ w1, const S* __restrict__ w2,
    const S* __restrict__ shift, float* prev,
    const i32* __restrict__ row_seq, const i32* __restrict__ cu,
    const i32* __restrict__ q_start, const i32* __restrict__ sslot,
    float eps, int W) {
  // last == nullptr: every chunk is a single row (a decode step); the row's
  // norm goes straight into its state slot, each element read before it is
  // overwritten by the same thread.
  __shared__ float red[8];
  const int t = blockIdx.x;
  const int b = row_seq[t];
  const int r0 = cu[b];
  const bool first = (t == r0);
  const bool is_last = (t == cu[b + 1] - 1);
  const int pos = q_start[b] + (t - r0);
  const float* xr = x + (size_t)t * W;
  const float* xp = xr - W;  // previous row, only touched when !first
  const bool need_prev_row = shift && !first;
  float ss[2] = {0.f, 0.f};
  for (int i = threadIdx.x * V; i < W; i += 256 * V) {
    float xv[4], pv4[4];
    ldv<float, V>(xr + i, xv);
#pragma unroll
    for (int j = 0; j < V; ++j) ss[0] += xv[j] * xv[j];
    if (need_prev_row) {
      ldv<float, V>(xp + i, pv4);
#pragma unroll
      for (int j = 0; j < V; ++j) ss[1] += pv4[j] * pv4[j];
    }
  }
  block_sum<2>(ss, red);
  const float r = 1.0f / sqrtf(ss[0] / (float)W + eps);
  const float rp = 1.0f / sqrtf(ss[1] / (float)W + eps);
  const float* pv = (shift && first && pos > 0)
                        ? prev + (size_t)sslot[b] * W : nullptr;
  for (int i = threadIdx.x * V; i < W; i += 256 * V) {
    float xv[4], g1[4], a[4], o[4], tmp[4];
    ldv<float, V>(xr + i, xv);
    ldv<S, V>(w1 + i, g1);
#pragma unroll
    for (int j = 0; j < V; ++j) { g1[j] += 1.0f; a[j] = xv[j] * r * g1[j]; }
    stv<S, V>(a_out + (size_t)t * W + i, a);
    if (b_out) {
      ldv<S, V>(w2 + i, tmp);
#pragma unroll
      for (int j = 0; j < V; ++j) o[j] = xv[j] * r * (1.0f + tmp[j]);
      stv<S, V>(b_out + (size_t)t * W + i, o);
    }
    if (shift) {
      float ap[4] = {0.f, 0.f, 0.f, 0.f};
      if (need_prev_row) {
        ldv<float, V>(xp + i, tmp);
#pragma unroll
        for (int j = 0; j < V; ++j) ap[j] = tmp[j] * rp * g1[j];
      } else if (pv) {
        ldv<float, V>(pv + i, ap);
      }
      ldv<S, V>(shift + i, tmp);
#pragma unroll
      for (int j = 0; j < V; ++j) o[j] = a[j] + (ap[j] - a[j]) * tmp[j];
      stv<S, V>(s_out + (size_t)t * W + i, o);
      if (is_last)
        stv<float, V>(last ? last + (size_t)b * W + i
                           : prev + (size_t)sslot[b] * W + i, a);
    }
  }
}

__global__ void __launch_bounds__(256) scatter_state_kernel(
    float* __restrict__ prev, const float* __restrict__ last,
    const i32* __restrict__ sslot, const i32* __restrict__ cu, int W) {
  const int b = blockIdx.x;
  if (cu[b + 1] == cu[b]) return;
  float* dst = prev + (size_t)sslot[b] * W;
  const float* src = last + (size_t)b * W;
  for (int i = threadIdx.x; i < W; i += 256) dst[i] = src[i];
}

template <typename S>
__global__ void __launch_bounds__(256) norm_rows_kernel(
    S* __restrict__ out, const float* __restrict__ x, const S* __restrict__ w,
    const i32* __restrict__ rows, float eps, int W, int one_plus) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * W;
  float ss[1] = {0.f};
  for (int i = threadIdx.x; i < W; i += 256) ss[0] += xr[i] * xr[i];
  block_sum<1>(ss, red);
  const float rs = 1.0f / sqrtf(ss[0] / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const float g = ldf<S>(w + i) + (one_plus ? 1.0f : 0.f);
    stf<S>(out + (size_t)r * W + i, xr[i] * rs * g);
  }
}

// One wave per (row, head): RMS over dv of fp32 o, * weight, * silu(gate)
// (SIG: * sigmoid(gate)).
template <typename S, int V, bool SIG>
__global__ void __launch_bounds__(256) headnorm_gate_kernel(
    S* __restrict__ out, const float* __restrict__ o, const S* __restrict__ g,
    const S* __restrict__ w, float eps, int n_rh, int H, int dv, i64 ldg) {
  const int rh = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (rh >= n_rh) return;
  const int lane = threadIdx.x & 63;
  const int t = rh / H, h = rh % H;
  const float* orow = o + ((size_t)t * H + h) * dv;
  float ss = 0.f;
  for (int d = lane * V; d < dv; d += 64 * V) {
    float ov[4];
    ldv<float, V>(orow + d, ov);
#pragma unroll
    for (int j = 0; j < V; ++j) ss += ov[j] * ov[j];
  }
  ss = wave_sum_f32(ss);
  const float rs = 1.0f / sqrtf(ss / (float)dv + eps);
  const S* grow = g + (size_t)t * ldg + (size_t)h * dv;
  for (int d = lane * V; d < dv; d += 64 * V) {
    float ov[4], gv[4], wv[4] = {1.f, 1.f, 1.f, 1.f}, r[4];
    ldv<float, V>(orow + d, ov);
    ldv<S, V>(grow + d, gv);
    if (w) ldv<S, V>(w + d, wv);
#pragma unroll
    for (int j = 0; j < V; ++j)
      r[j] = ov[j] * rs * wv[j] * ((SIG ? 1.0f : gv[j]) / (1.0f + expf(-gv[j])));
    stv<S, V>(out + ((size_t)t * H + h) * dv + d, r);
  }
}

template <typename S, int V>
__global__ void __launch_bounds__(256) polynorm_kernel(
    S* __restrict__ out, const S* __restrict__ z, const float* __restrict__ coef,
    float eps, int F, i64 ldz) {
  __shared__ float red[12];
  const int t = blockIdx.x;
  const S* zr = z + (size_t)t * ldz;
  float s[3] = {0.f, 0.f, 0.f};
  for (int i = threadIdx.x * V; i < F; i += 256 * V) {
    float v[4];
    ldv<S, V>(zr + i, v);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float v2 = v[j] * v[j];
      s[0] += v2;
      s[1] += v2 * v2;
      s[2] += v2 * v2 * v2;
    }
  }
  block_sum<3>(s, red);
  const float r1 = 1.0f / sqrtf(s[0] / (float)F + eps);
  const float r2 = 1.0f / sqrtf(s[1] / (float)F + eps);
  const float r3 = 1.0f / sqrtf(s[2] / (float)F + eps);
  const float c0 = coef[0], c1 = coef[1], c2 = coef[2], c3 = coef[3];
  for (int i = threadIdx.x * V; i < F; i += 256 * V) {
    float v[4], o[4];
    ldv<S, V>(zr + i, v);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float v2 = v[j] * v[j];
      o[j] = c0 * (v[j] * r1) + c1 * (v2 * r2) + c2 * (v2 * v[j] * r3) + c3;
    }
    stv<S, V>(out + (size_t)t * F + i, o);
  }
}

template <typename S, int V>
__global__ void __launch_bounds__(256) gated_residual_kernel(
    float* __restrict__ x, const S* __restrict__ a, float sa,
    const S* __restrict__ b, float sb, const S* __restrict__ g1, i64 ldg1,
    const float* __restrict__ b1, const S* __restrict__ m,
    const S* __restrict__ g2, i64 ldg2, const float* __restrict__ b2,
    int T, int W) {
  const i64 n = (i64)T * W;
  for (i64 i = ((i64)blockIdx.x * 256 + threadIdx.x) * V; i < n;
       i += (i64)gridDim.x * 256 * V) {
    const int t = (int)(i / W), c = (int)(i % W);
    float xv[4], av[4], bv[4] = {0.f, 0.f, 0.f, 0.f}, gv[4], bias[4], mv[4];
    ldv<float, V>(x + i, xv);
    ldv<S, V>(a + i, av);
    if (b) ldv<S, V>(b + i, bv);
    ldv<S, V>(g1 + (size_t)t * ldg1 + c, gv);
    ldv<float, V>(b1 + c, bias);
#pragma unroll
    for (int j = 0; j < V; ++j)
      xv[j] += (sa * av[j] + sb * bv[j]) / (1.0f + expf(-(gv[j] + bias[j])));
    if (m) {
      ldv<S, V>(m + i, mv);
      ldv<S, V>(g2 + (size_t)t * ldg2 + c, gv);
      ldv<float, V>(b2 + c, bias);
#pragma unroll
      for (int j = 0; j < V; ++j)
        xv[j] += mv[j] / (1.0f + expf(-(gv[j] + bias[j])));
    }
    stv<float, V>(x + i, xv);
  }
}

template <typename S>
__global__ void __launch_bounds__(256) softcap_kernel(
    float* __restrict__ out, const S* __restrict__ in, float cap, i64 n) {
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    const float v = ldf<S>(in + i);
    out[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}

// fp32 rows -> storage dtype (the projections' input when sublayers read the
// residual itself).
template <typename S>
__global__ void __launch_bounds__(256) cast_rows_kernel(
    S* __restrict__ out, const float* __restrict__ x, i64 n) {
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256)
    stf<S>(out + i, x[i]);
}

// Norm on a sublayer's OUTPUT, then the residual add:
//   u = y (+ bias);  x += u / sqrt(mean(u^2) + eps) * w;  h = S(x)
// y is [T, W] in Y (storage dtype or fp32), x the fp32 residual, h an
// optional copy of the new residual row in the storage dtype.
template <typename S, typename Y, int V>
__global__ void __launch_bounds__(256) norm_residual_kernel(
    float* __restrict__ x, S* __restrict__ h, const Y* __restrict__ y,
    i64 ldy, const S* __restrict__ bias, const S* __restrict__ w, float eps,
    int W) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const Y* yr = y + (size_t)t * ldy;
  float ss[1] = {0.f};
  for (int i = threadIdx.x * V; i < W; i += 256 * V) {
    float u[4], bv[4] = {0.f, 0.f, 0.f, 0.f};
    ldv<Y, V>(yr + i, u);
    if (bias) ldv<S, V>(bias + i, bv);
#pragma unroll
    for (int j = 0; j < V; ++j) { u[j] += bv[j]; ss[0] += u[j] * u[j]; }
  }
  block_sum<1>(ss, red);
  const float rs = 1.0f / sqrtf(ss[0] / (float)W + eps);
  float* xr = x + (size_t)t * W;
  for (int i = threadIdx.x * V; i < W; i += 256 * V) {
    float u[4], bv[4] = {0.f, 0.f, 0.f, 0.f}, wv[4], xv[4];
    ldv<Y, V>(yr + i, u);
    if (bias) ldv<S, V>(bias + i, bv);
    ldv<S, V>(w + i, wv);
    ldv<float, V>(xr + i, xv);
#pragma unroll
    for (int j = 0; j < V; ++j) xv[j] += (u[j] + bv[j]) * rs * wv[j];
    stv<float, V>(xr + i, xv);
    if (h) stv<S, V>(h + (size_t)t * W + i, xv);
  }
}

// Gated linear unit over rows of [gate | up]:
//   out[r, i] = act(g[r, i] + bg[i]) * (u[r, i] + bu[i]) * rw[r]
// act: 0 SiLU, 1 ReLU, 2 tanh-GELU.  Biases and the per-row weight rw (fp32,
// e.g. a router weight per (token, expert) row) are optional.  Row r sits at
// (r / rg) * ld + (r % rg) * ld_in, so rg units laid side by side in one
// matrix row (experts of one token) are rows of their own.
template <typename S, int ACT, int V>
__global__ void __launch_bounds__(256) glu_kernel(
    S* __restrict__ out, i64 ldo, i64 ldo_in, const S* __restrict__ g,
    const S* __restrict__ u, i64 ldi, i64 ldi_in, int rg,
    const S* __restrict__ bg, const S* __restrict__ bu,
    const float* __restrict__ rw, i64 R, int F, float limit) {
  const int FV = F / V;
  const i64 n = R * FV;
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < n;
       i += (i64)gridDim.x * 256) {
    const i64 r = i / FV;
    const int c = (int)(i % FV) * V;
    const i64 ri = (r / rg) * ldi + (r % rg) * ldi_in;
    float a[4], b[4], ba[4] = {0.f, 0.f, 0.f, 0.f}, bb[4] = {0.f, 0.f, 0.f, 0.f};
    ldv<S, V>(g + ri + c, a);
    ldv<S, V>(u + ri + c, b);
    if (bg) ldv<S, V>(bg + c, ba);
    if (bu) ldv<S, V>(bu + c, bb);
    const float wr = rw ? rw[r] : 1.0f;
    float o[4];
#pragma unroll
    for (int j = 0; j < V; ++j) {
      float av = a[j] + ba[j];
      float uv = b[j] + bb[j];
      if (ACT == 0) av = av / (1.0f + expf(-av));
      else if (ACT == 1) av = fmaxf(av, 0.f);
      else if (ACT == 2)
        av = 0.5f * av * (1.0f + tanhf(0.7978845608028654f *
                                       (av + 0.044715f * av * av * av)));
      else {   // clamped unit: min(g, L) sigmoid(1.702 g) (clamp(u, -L, L) + 1)
        av = fminf(av, limit);
        av = av / (1.0f + expf(-1.702f * av));
        uv = fminf(fmaxf(uv, -limit), limit) + 1.0f;
      }
      o[j] = av * uv * wr;
    }
    stv<S, V>(out + (r / rg) * ldo + (r % rg) * ldo_in + c, o);
  }
}

// Sigmoid router with score correction and group-limited top-k, one wave per
// token.  z [T, E] fp32 logits; s = sigmoid(z); choice = s + corr.  With
// n_groups > 0 the experts form n_groups equal groups of neighbours, a
// group's score is the sum of its two largest choice scores, and experts
// outside the best `keep` groups cannot be chosen.  The `top` largest choice
// scores win (ties: lower index); weights = s / (sum of chosen s + 1e-20) *
// scale.  Outputs idx [T, top] i32, wts [T, top] fp32 and, optionally, the
// dense form wd [T, E] fp32 (zero for experts not chosen).
__global__ void __launch_bounds__(64) moe_route_kernel(
    i32* __restrict__ idx, float* __restrict__ wts, float* __restrict__ wd,
    const float* __restrict__ z, const float* __restrict__ corr, int E,
    int top, int n_groups, int keep, float scale, int softmax, int renorm) {
  extern __shared__ float sh[];
  float* sig = sh;             // [E]
  float* choice = sh + E;      // [E]
  float* gsc = sh + 2 * E;     // [n_groups]
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* zr = z + (size_t)t * E;
  float zmax = 0.f, zinv = 1.f;
  if (softmax) {       // scores are softmax(z) over all experts
    zmax = -INFINITY;
    for (int e = lane; e < E; e += 64) zmax = fmaxf(zmax, zr[e]);
    zmax = wave_max_f32(zmax);
    float zs = 0.f;
    for (int e = lane; e < E; e += 64) zs += expf(zr[e] - zmax);
    zinv = 1.0f / wave_sum_f32(zs);
  }
  for (int e = lane; e < E; e += 64) {
    const float s = softmax ? expf(zr[e] - zmax) * zinv
                            : 1.0f / (1.0f + expf(-zr[e]));
    sig[e] = s;
    choice[e] = s + (corr ? corr[e] : 0.f);
    if (wd) wd[(size_t)t * E + e] = 0.f;
  }
  __syncthreads();
  if (n_groups > 0 && keep < n_groups) {
    const int size = E / n_groups;
    for (int g = lane; g < n_groups; g += 64) {
      float a = -INFINITY, b = -INFINITY;   // largest, second largest
      for (int m = 0; m < size; ++m) {
        const float c = choice[g * size + m];
        if (c > a) { b = a; a = c; }
        else if (c > b) b = c;
      }
      gsc[g] = size > 1 ? a + b : a;
    }
    __syncthreads();
    for (int g = lane; g < n_groups; g += 64) {
      const float mine = gsc[g];
      int rank = 0;
      for (int o = 0; o < n_groups; ++o)
        rank += (gsc[o] > mine || (gsc[o] == mine && o < g)) ? 1 : 0;
      if (rank >= keep)
        for (int m = 0; m < size; ++m) choice[g * size + m] = -INFINITY;
    }
    __syncthreads();
  }
  float total = 0.f;
  for (int r = 0; r < top; ++r) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float c = choice[e];
      if (c > bv) { bv = c; bi = e; }   // ascending e: first of equals stays
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi >= E) bi = r < E ? r : 0;    // fewer candidates than `top`
    total += sig[bi];
    if (lane == 0) {
      idx[(size_t)t * top + r] = bi;
      wts[(size_t)t * top + r] = sig[bi];
      choice[bi] = -INFINITY;
    }
    __syncthreads();
  }
  const float inv = renorm ? scale / (total + 1e-20f) : scale;
  for (int r = lane; r < top; r += 64) {
    const float w = wts[(size_t)t * top + r] * inv;
    wts[(size_t)t * top + r] = w;
    if (wd) wd[(size_t)t * E + idx[(size_t)t * top + r]] = w;
  }
}

// y[t] = sum_r wts[t, r] * ys[pos[t*top + r]] (+ shared[t]) in fp32, the sum
// taken in the order r = 0 .. top-1.  ys rows sit in expert-sorted order; pos
// is the inverse of that sort.
template <typename S>
__global__ void __launch_bounds__(256) moe_combine_kernel(
    float* __restrict__ y, const S* __restrict__ ys,
    const i32* __restrict__ pos, const float* __restrict__ wts,
    const S* __restrict__ shared, int top, int W) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < W; i += 256) {
    float acc = shared ? ldf<S>(shared + (size_t)t * W + i) : 0.f;
    for (int r = 0; r < top; ++r)
      acc += wts[(size_t)t * top + r] *
             ldf<S>(ys + (size_t)pos[(size_t)t * top + r] * W + i);
    y[(size_t)t * W + i] = acc;
  }
}

template <typename... P>
inline bool aligned16(P... p) {
  return ((((uintptr_t)p) % 16 == 0) && ...);
}

inline int grid_for(i64 n) {
  i64 g = (n + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

}  // namespace

#define MIX_DISPATCH(dt, CALL_BF, CALL_F32) \
  do {                                      \
    if ((dt) == 0) { CALL_BF; }             \
    else if ((dt) == 1) { CALL_F32; }       \
    else return 9002;                       \
  } while (0)

AF_EXPORT int afm_embed(void* out, const void* table, const void* ids,
                        const void* add, float scale, int T, int W, int dt,
                        void* stream) {
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  MIX_DISPATCH(dt,
      (embed_kernel<u16><<<T, 256, 0, s>>>((float*)out, (const u16*)table,
          (const i32*)ids, (const float*)add, scale, W)),
      (embed_kernel<float><<<T, 256, 0, s>>>((float*)out, (const float*)table,
          (const i32*)ids, (const float*)add, scale, W)));
  return af_last_err();
}

AF_EXPORT int afm_add_rows(void* x, const void* other, const void* vec, int T,
                           int W, void* stream) {
  if (T == 0) return 0;
  const i64 n = (i64)T * W;
  add_rows_kernel<<<grid_for(n), 256, 0, (hipStream_t)stream>>>(
      (float*)x, (const float*)other, (const float*)vec, n, W);
  return af_last_err();
}

AF_EXPORT int afm_dual_norm_shift(
    void* a, void* s_out, void* b, void* last, const void* x, const void* w1,
    const void* w2, const void* shift, const void* prev, const void* row_seq,
    const void* cu, const void* q_start, const void* sslot, float eps, int T,
    int W, int dt, void* stream) {
  if (T == 0) return 0;
  if (shift && !prev) return 9003;
  if ((b == nullptr) != (w2 == nullptr)) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = W % 4 == 0 && aligned16(a, s_out, b, last, x, w1) &&
                   aligned16(w2, shift, prev);
#define DNS(ST, V)                                                            \
  dual_norm_shift_kernel<ST, V><<<T, 256, 0, s>>>((ST*)a, (ST*)s_out, (ST*)b, \
      (float*)last, (const float*)x, (const ST*)w1, (const ST*)w2,            \
      (const ST*)shift, (float*)prev, (const i32*)row_seq,                    \
      (const i32*)cu, (const i32*)q_start, (const i32*)sslot, eps, W)
  if (vec) MIX_DISPATCH(dt, (DNS(u16, 4)), (DNS(float, 4)));
  else MIX_DISPATCH(dt, (DNS(u16, 1)), (DNS(float, 1)));
#undef DNS
  return af_last_err();
}

AF_EXPORT int afm_scatter_state(void* prev, const void* last,
                                const void* sslot, const void* cu, int B,
                                int W, void* stream) {
  if (B == 0) return 0;
  scatter_state_kernel<<<B, 256, 0, (hipStream_t)stream>>>(
      (float*)prev, (const float*)last, (const i32*)sslot, (const i32*)cu, W);
  return af_last_err();
}

AF_EXPORT int afm_norm_rows(void* out, const void* x, const void* w,
                            const void* rows, float eps, int R, int W,
                            int one_plus, int dt, void* stream) {
  if (R == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  MIX_DISPATCH(dt,
      (norm_rows_kernel<u16><<<R, 256, 0, s>>>((u16*)out, (const float*)x,
          (const u16*)w, (const i32*)rows, eps, W, one_plus)),
      (norm_rows_kernel<float><<<R, 256, 0, s>>>((float*)out, (const float*)x,
          (const float*)w, (const i32*)rows, eps, W, one_plus)));
  return af_last_err();
}

AF_EXPORT int afm_headnorm_gate(void* out, const void* o, const void* g,
                                const void* w, float eps, int T, int H, int dv,
                                i64 ldg, int gate_act, int dt, void* stream) {
  if (T == 0) return 0;
  const int n_rh = T * H;
  const int grid = (n_rh + 3) / 4;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = dv % 4 == 0 && ldg % 4 == 0 && aligned16(out, o, g, w);
#define HG(ST, V, SG)                                                       \
  headnorm_gate_kernel<ST, V, SG><<<grid, 256, 0, s>>>((ST*)out,            \
      (const float*)o, (const ST*)g, (const ST*)w, eps, n_rh, H, dv, ldg)
  if (gate_act == 1) {
    if (vec) MIX_DISPATCH(dt, (HG(u16, 4, true)), (HG(float, 4, true)));
    else MIX_DISPATCH(dt, (HG(u16, 1, true)), (HG(float, 1, true)));
  } else {
    if (vec) MIX_DISPATCH(dt, (HG(u16, 4, false)), (HG(float, 4, false)));
    else MIX_DISPATCH(dt, (HG(u16, 1, false)), (HG(float, 1, false)));
  }
#undef HG
  return af_last_err();
}

AF_EXPORT int afm_polynorm(void* out, const void* z, const void* coef,
                           float eps, int T, int F, i64 ldz, int dt,
                           void* stream) {
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = F % 4 == 0 && ldz % 4 == 0 && aligned16(out, z);
#define PN(ST, V)                                                     \
  polynorm_kernel<ST, V><<<T, 256, 0, s>>>((ST*)out, (const ST*)z,    \
      (const float*)coef, eps, F, ldz)
  if (vec) MIX_DISPATCH(dt, (PN(u16, 4)), (PN(float, 4)));
  else MIX_DISPATCH(dt, (PN(u16, 1)), (PN(float, 1)));
#undef PN
  return af_last_err();
}

AF_EXPORT int afm_gated_residual(
    void* x, const void* a, float sa, const void* b, float sb, const void* g1,
    i64 ldg1, const void* b1, const void* m, const void* g2, i64 ldg2,
    const void* b2, int T, int W, int dt, void* stream) {
  if (T == 0) return 0;
  if (m && (!g2 || !b2)) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = W % 4 == 0 && ldg1 % 4 == 0 && ldg2 % 4 == 0 &&
                   aligned16(x, a, b, g1, b1, m) && aligned16(g2, b2);
  const int grid = grid_for((i64)T * W / (vec ? 4 : 1));
#define GR(ST, V)                                                          \
  gated_residual_kernel<ST, V><<<grid, 256, 0, s>>>((float*)x,             \
      (const ST*)a, sa, (const ST*)b, sb, (const ST*)g1, ldg1,             \
      (const float*)b1, (const ST*)m, (const ST*)g2, ldg2, (const float*)b2, \
      T, W)
  if (vec) MIX_DISPATCH(dt, (GR(u16, 4)), (GR(float, 4)));
  else MIX_DISPATCH(dt, (GR(u16, 1)), (GR(float, 1)));
#undef GR
  return af_last_err();
}

AF_EXPORT int afm_softcap(void* out, const void* in, float cap, i64 n, int dt,
                          void* stream) {
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  MIX_DISPATCH(dt,
      (softcap_kernel<u16><<<grid_for(n), 256, 0, s>>>((float*)out,
          (const u16*)in, cap, n)),
      (softcap_kernel<float><<<grid_for(n), 256, 0, s>>>((float*)out,
          (const float*)in, cap, n)));
  return af_last_err();
}

AF_EXPORT int afm_cast_rows(void* out, const void* x, i64 n, int dt,
                            void* stream) {
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  MIX_DISPATCH(dt,
      (cast_rows_kernel<u16><<<grid_for(n), 256, 0, s>>>((u16*)out,
          (const float*)x, n)),
      (cast_rows_kernel<float><<<grid_for(n), 256, 0, s>>>((float*)out,
          (const float*)x, n)));
  return af_last_err();
}

// y_f32 != 0: y holds fp32 whatever the storage dtype.
AF_EXPORT int afm_norm_residual(void* x, void* h, const void* y, i64 ldy,
                                int y_f32, const void* bias, const void* w,
                                float eps, int T, int W, int dt,
                                void* stream) {
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = W % 4 == 0 && ldy % 4 == 0 && aligned16(x, h, y, bias, w);
#define NR(ST, YT)                                                          \
  do {                                                                      \
    if (vec)                                                                \
      norm_residual_kernel<ST, YT, 4><<<T, 256, 0, s>>>((float*)x, (ST*)h,  \
          (const YT*)y, ldy, (const ST*)bias, (const ST*)w, eps, W);        \
    else                                                                    \
      norm_residual_kernel<ST, YT, 1><<<T, 256, 0, s>>>((float*)x, (ST*)h,  \
          (const YT*)y, ldy, (const ST*)bias, (const ST*)w, eps, W);        \
  } while (0)
  if (dt == 0) { if (y_f32) NR(u16, float); else NR(u16, u16); }
  else if (dt == 1) NR(float, float);
  else return 9002;
#undef NR
  return af_last_err();
}

AF_EXPORT int afm_glu(void* out, i64 ldo, i64 ldo_in, const void* g,
                      const void* u, i64 ldi, i64 ldi_in, int rg,
                      const void* bg, const void* bu, const void* rw, i64 R,
                      int F, int act, float limit, int dt, void* stream) {
  if (R == 0 || F == 0) return 0;
  if (act < 0 || act > 3 || rg < 1) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = F % 4 == 0 && ldo % 4 == 0 && ldo_in % 4 == 0 &&
                   ldi % 4 == 0 && ldi_in % 4 == 0 &&
                   aligned16(out, g, u, bg, bu);
  const int grid = grid_for(R * F / (vec ? 4 : 1));
#define GLU(ST, A)                                                         \
  do {                                                                     \
    if (vec)                                                               \
      glu_kernel<ST, A, 4><<<grid, 256, 0, s>>>((ST*)out, ldo, ldo_in,     \
          (const ST*)g, (const ST*)u, ldi, ldi_in, rg, (const ST*)bg,      \
          (const ST*)bu, (const float*)rw, R, F, limit);                          \
    else                                                                   \
      glu_kernel<ST, A, 1><<<grid, 256, 0, s>>>((ST*)out, ldo, ldo_in,     \
          (const ST*)g, (const ST*)u, ldi, ldi_in, rg, (const ST*)bg,      \
          (const ST*)bu, (const float*)rw, R, F, limit);                          \
  } while (0)
#define GLU_ACT(ST)                                   \
  do {                                                \
    if (act == 0) GLU(ST, 0);                         \
    else if (act == 1) GLU(ST, 1);                    \
    else if (act == 2) GLU(ST, 2);                    \
    else GLU(ST, 3);                                  \
  } while (0)
  MIX_DISPATCH(dt, GLU_ACT(u16), GLU_ACT(float));
#undef GLU_ACT
#undef GLU
  return af_last_err();
}

AF_EXPORT int afm_moe_route(void* idx, void* wts, void* wd, const void* z,
                            const void* corr, int T, int E, int top,
                            int n_groups, int keep, float scale, int softmax,
                            int renorm, void* stream) {
  if (T == 0) return 0;
  if (E < 1 || top < 1 || top > E) return 9003;
  if (n_groups > 0 && (E % n_groups != 0 || keep < 1)) return 9003;
  const size_t sm = (size_t)(2 * E + (n_groups > 0 ? n_groups : 0)) *
                    sizeof(float);
  if (sm > 60000) return 9004;
  moe_route_kernel<<<T, 64, sm, (hipStream_t)stream>>>(
      (i32*)idx, (float*)wts, (float*)wd, (const float*)z, (const float*)corr,
      E, top, n_groups, keep, scale, softmax, renorm);
  return af_last_err();
}

AF_EXPORT int afm_moe_combine(void* y, const void* ys, const void* pos,
                              const void* wts, const void* shared, int T,
                              int top, int W, int dt, void* stream) {
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  MIX_DISPATCH(dt,
      (moe_combine_kernel<u16><<<T, 256, 0, s>>>((float*)y, (const u16*)ys,
          (const i32*)pos, (const float*)wts, (const u16*)shared, top, W)),
      (moe_combine_kernel<float><<<T, 256, 0, s>>>((float*)y, (const float*)ys,
          (const i32*)pos, (const float*)wts, (const float*)shared, top, W)));
  return af_last_err();
}
