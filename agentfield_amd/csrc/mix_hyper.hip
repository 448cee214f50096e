// Glue of hyper-connected decoders: several fp32 residual streams per token
// mixed by small learned matrices, an RMSNorm and a short causal convolution
// in front of every sublayer, and the row-wise steps of latent attention
// (latent norm, interleaved rotary positions, cache append, query assembly,
// gated head outputs).
//
// Storage dtype S is bf16 (raw u16) or fp32.  The streams, norm statistics,
// convolution inputs and sums, angles and gates are fp32; S is what the
// projections read and write.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// V consecutive elements as floats (V = 4: one 8- or 16-byte access)
template <typename S, int V>
__device__ __forceinline__ void ldv(const S* p, float (&o)[4]) {
  if constexpr (V == 4) {
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
__device__ __forceinline__ void stv(S* p, const float (&o)[4]) {
  if constexpr (V == 4) {
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

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum_f32(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  const float s = red[0] + red[1] + red[2] + red[3];
  __syncthreads();
  return s;
}

// the same for NT threads (a multiple of 64, at most 1024), fixed order
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum_f32(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) s += red[w];
  __syncthreads();
  return s;
}

// ------------------------------------------------------------ embedding
// x[t, s, :] = table[ids[t]] for every stream s.
template <typename S>
__global__ void __launch_bounds__(256) embed_streams_kernel(
    float* __restrict__ x, const S* __restrict__ table,
    const i32* __restrict__ ids, int ns, int W) {
  const int t = blockIdx.x;
  const S* row = table + (size_t)ids[t] * W;
  float* xr = x + (size_t)t * ns * W;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = ldf<S>(row + c);
    for (int s = 0; s < ns; ++s) xr[(size_t)s * W + c] = v;
  }
}

// ------------------------------------------------------------ stream step
// One workgroup per token row.  With y: the streams take the sublayer output
// in, all at once from the old ones:
//     x_r <- sum_s mix[s, r] x_s + out[r] y            (r = 0..ns-1)
// With in: the next sublayer's input is read out, u = sum_r in[r] x_r, and
// left in `n` either as it is (norm_mode 0) or as u / rms(u) * (1 + w)
// (norm_mode 1).  MS bounds the stream count; V columns per access.
//
// With a convolution tail (steps of one row per sequence, row t = sequence
// t): the normed row goes straight through the input convolution, h = n +
// sum_j w[:, j] n_(t - (taps-1-j)) with the earlier inputs taken from the
// sequence's slot, h leaves in the storage dtype, and the slot moves on by
// one input; `n` is then scratch.
struct ConvTail {
  const void* w;       // [W, taps] storage dtype, null: no tail
  float* state;        // [slots, max(taps-1, 1), W]
  const i32* sslot;    // [T]
  const i32* pos;      // [T] position of the row
  void* h;             // [T, W] storage dtype
  int taps;
};

// NT threads per row: 256 when rows are plenty, 1024 for steps of few rows,
// whose time is the chain of dependent loads of one workgroup's iterations.
template <typename S, int MS, int V, int NT>
__global__ void __launch_bounds__(NT) hyper_step_kernel(
    float* __restrict__ x, const S* __restrict__ y, i64 ldy,
    const float* __restrict__ mixm, const float* __restrict__ outv,
    const float* __restrict__ inv, const S* __restrict__ normw, float eps,
    float* __restrict__ n, int ns, int W, int norm_mode, ConvTail ct) {
  __shared__ float s_mix[MS * MS], s_in[MS], s_out[MS], red[NT / 64];
  const int t = blockIdx.x;
  if (threadIdx.x < MS * MS) {
    const int s = threadIdx.x / MS, r = threadIdx.x % MS;
    s_mix[threadIdx.x] = (y && s < ns && r < ns) ? mixm[s * ns + r] : 0.f;
  }
  if (threadIdx.x < MS) {
    s_in[threadIdx.x] = (inv && (int)threadIdx.x < ns) ? inv[threadIdx.x] : 0.f;
    s_out[threadIdx.x] = (y && (int)threadIdx.x < ns) ? outv[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float* xr = x + (size_t)t * ns * W;
  float* nr = n ? n + (size_t)t * W : nullptr;
  float ss = 0.f;
  // the first KEEP column groups of a thread stay in registers across the
  // row reduction; wider rows go through `n`
  constexpr int KEEP = 4;
  float held[KEEP][4];
  int it = 0;
  for (int c = threadIdx.x * V; c < W; c += NT * V, ++it) {
    float xs[MS][4];
#pragma unroll
    for (int s = 0; s < MS; ++s)
      if (s < ns) ldv<float, V>(xr + (size_t)s * W + c, xs[s]);
    if (y) {
      float yv[4], nw[MS][4];
      ldv<S, V>(y + (size_t)t * ldy + c, yv);
#pragma unroll
      for (int r = 0; r < MS; ++r) {
        if (r >= ns) continue;
#pragma unroll
        for (int j = 0; j < V; ++j) nw[r][j] = s_out[r] * yv[j];
#pragma unroll
        for (int s = 0; s < MS; ++s)
          if (s < ns) {
#pragma unroll
            for (int j = 0; j < V; ++j) nw[r][j] += s_mix[s * MS + r] * xs[s][j];
          }
      }
#pragma unroll
      for (int r = 0; r < MS; ++r)
        if (r < ns) {
#pragma unroll
          for (int j = 0; j < V; ++j) xs[r][j] = nw[r][j];
          stv<float, V>(xr + (size_t)r * W + c, nw[r]);
        }
    }
    if (inv) {
      float u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < MS; ++r)
        if (r < ns) {
#pragma unroll
          for (int j = 0; j < V; ++j) u[j] += s_in[r] * xs[r][j];
        }
#pragma unroll
      for (int j = 0; j < V; ++j) ss += u[j] * u[j];
      if (norm_mode == 0 || it >= KEEP) stv<float, V>(nr + c, u);
#pragma unroll
      for (int k = 0; k < KEEP; ++k)
        if (k == it) {
#pragma unroll
          for (int j = 0; j < V; ++j) held[k][j] = u[j];
        }
    }
  }
  if (!inv || norm_mode == 0) return;
  const float rinv = 1.0f / sqrtf(block_sum<NT>(ss, red) / (float)W + eps);
  const int tail_pos = ct.w ? ct.pos[t] : 0;
  const int tail_slot = ct.w ? ct.sslot[t] : 0;
  it = 0;
  for (int c = threadIdx.x * V; c < W; c += NT * V, ++it) {
    float u[4], w4[4];
    if (it >= KEEP) ldv<float, V>(nr + c, u);   // columns this thread wrote
#pragma unroll
    for (int k = 0; k < KEEP; ++k)
      if (k == it) {
#pragma unroll
        for (int j = 0; j < V; ++j) u[j] = held[k][j];
      }
    ldv<S, V>(normw + c, w4);
#pragma unroll
    for (int j = 0; j < V; ++j) u[j] *= rinv * (1.0f + w4[j]);
    if (!ct.w) {
      stv<float, V>(nr + c, u);
      continue;
    }
    const int hist = ct.taps - 1;
    const int p = tail_pos;
    float* st = ct.state + (size_t)tail_slot * (hist > 0 ? hist : 1) * W;
    const S* cw = (const S*)ct.w + (size_t)c * ct.taps;
    float acc[4];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = u[j] + ldf<S>(cw + j * ct.taps + hist) * u[j];
    // place i of the slot holds the input of position p - hist + i; walking
    // from the oldest, each is weighed by tap i and moved one place down
    for (int i = 0; i < hist; ++i) {
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (p - hist + i >= 0) ldv<float, V>(st + (size_t)i * W + c, v);
#pragma unroll
      for (int j = 0; j < V; ++j) acc[j] += ldf<S>(cw + j * ct.taps + i) * v[j];
      if (i > 0) stv<float, V>(st + (size_t)(i - 1) * W + c, v);
    }
    if (hist > 0) stv<float, V>(st + (size_t)(hist - 1) * W + c, u);
    stv<S, V>((S*)ct.h + (size_t)t * W + c, acc);
  }
}

// ------------------------------------------------- input convolution
// h[t, c] = n[t, c] + sum_j w[c, j] n[t - (taps-1-j), c]: a causal depthwise
// convolution added to its own input.  Rows before the chunk come from the
// sequence's slot of `state` [slots, taps-1, W] fp32 (oldest first), rows
// before position 0 are zero.  One workgroup per (row, 256 channels).
constexpr int CONV_ROWS = 8;   // consecutive rows per workgroup: a row's
                               // predecessors were just read by the same CU
constexpr int CONV_REGT = 8;   // taps whose weights stay in registers

template <typename S, int V>
__global__ void __launch_bounds__(256) canon_conv_kernel(
    S* __restrict__ h, const float* __restrict__ n, const S* __restrict__ w,
    const float* __restrict__ state, const i32* __restrict__ row_seq,
    const i32* __restrict__ cu, const i32* __restrict__ q_start,
    const i32* __restrict__ sslot, int T, int W, int taps) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * V;
  if (c >= W) return;
  const int hist = taps - 1;
  const S* cw = w + (size_t)c * taps;
  float wb[CONV_REGT][4];        // wb[k]: weight of the input k rows back
#pragma unroll
  for (int k = 0; k < CONV_REGT; ++k)
#pragma unroll
    for (int j = 0; j < V; ++j)
      wb[k][j] = k <= hist ? ldf<S>(cw + j * taps + hist - k) : 0.f;
  const int t0 = blockIdx.x * CONV_ROWS;
  const int t1 = min(T, t0 + CONV_ROWS);
  for (int t = t0; t < t1; ++t) {
    const int b = row_seq[t];
    const int r = t - cu[b];
    const int p = q_start[b] + r;
    const float* st = state + (size_t)sslot[b] * (hist > 0 ? hist : 1) * W;
    float cur[4], acc[4];
    ldv<float, V>(n + (size_t)t * W + c, cur);
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = cur[j] + wb[0][j] * cur[j];
#pragma unroll
    for (int k = 1; k < CONV_REGT; ++k) {
      if (k > hist || p - k < 0) break;       // before the sequence: zeros
      float v[4];
      if (r - k >= 0) ldv<float, V>(n + (size_t)(t - k) * W + c, v);
      else ldv<float, V>(st + (size_t)(hist + r - k) * W + c, v);
#pragma unroll
      for (int j = 0; j < V; ++j) acc[j] += wb[k][j] * v[j];
    }
    for (int k = CONV_REGT; k <= hist && p - k >= 0; ++k) {
      float v[4];
      if (r - k >= 0) ldv<float, V>(n + (size_t)(t - k) * W + c, v);
      else ldv<float, V>(st + (size_t)(hist + r - k) * W + c, v);
#pragma unroll
      for (int j = 0; j < V; ++j) acc[j] += ldf<S>(cw + j * taps + hist - k) * v[j];
    }
    stv<S, V>(h + (size_t)t * W + c, acc);
  }
}

// After the convolution: the slot keeps the sequence's last taps-1 inputs.
// A chunk shorter than that keeps the tail of the old content in front.
__global__ void __launch_bounds__(256) canon_state_kernel(
    float* __restrict__ state, const float* __restrict__ n,
    const i32* __restrict__ cu, const i32* __restrict__ q_start,
    const i32* __restrict__ sslot, int W, int taps) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int r0 = cu[b], len = cu[b + 1] - r0;
  const int hist = taps - 1;
  if (c >= W || len <= 0 || hist <= 0) return;
  float* st = state + (size_t)sslot[b] * hist * W;
  const int qs = q_start[b];
  for (int i = 0; i < hist; ++i) {
    const int rr = len - hist + i;           // chunk row kept in place i
    float v;
    if (qs + rr < 0) v = 0.f;
    else if (rr >= 0) v = n[(size_t)(r0 + rr) * W + c];
    else v = st[(size_t)(hist + rr) * W + c];     // = old place len + i > i
    st[(size_t)i * W + c] = v;
  }
}

// ------------------------------------------------------- latent attention
// One workgroup per row.  The down projection's row holds the latent (first
// R values) and one rotary key part (rd values); the latent is RMS-normed
// with a plain weight, the key part rotated, and [latent | key part] goes to
// the key pages [P, 1, page, R + rd] at `slot`.  The attention query of head
// h is [q in latent space (R, already in place) | rotate(q[t, h, dim:dim+rd])]:
// the kernel fills the rotary slices of qf [T, H, R + rd].  Rotation pairs
// element 2i with 2i+1 for i < rot/2, angle = position * inv_freq[i] in fp32.
template <typename S>
__global__ void __launch_bounds__(256) latent_prep_kernel(
    S* __restrict__ qf, S* __restrict__ kc, const S* __restrict__ q, i64 ldq,
    const S* __restrict__ dkv, i64 lddkv,
    const S* __restrict__ normw, const float* __restrict__ inv_freq,
    const i32* __restrict__ positions, const i64* __restrict__ slots,
    float eps, int T, int H, int dim, int rd, int R, int rot) {
  __shared__ float red[4];
  extern __shared__ float cs[];              // [rot/2] cos, [rot/2] sin
  const int t = blockIdx.x;
  const int half = rot / 2;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < half; i += 256) {
    float sn, c;
    sincosf(pos * inv_freq[i], &sn, &c);
    cs[i] = c;
    cs[half + i] = sn;
  }
  const S* dr = dkv + (size_t)t * lddkv;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += 256) {
    const float v = ldf<S>(dr + i);
    ss += v * v;
  }
  const float rinv = 1.0f / sqrtf(block_sum_256(ss, red) / (float)R + eps);
  const i64 sl = slots[t];
  const int dkc = R + rd;
  if (sl >= 0) {
    S* kr = kc + (size_t)sl * dkc;           // one K/V head: slot * row
    for (int i = threadIdx.x; i < R; i += 256)
      stf<S>(kr + i, ldf<S>(dr + i) * rinv * ldf<S>(normw + i));
    for (int i = threadIdx.x; i < rd; i += 256) {
      float v = ldf<S>(dr + R + i);
      if (i < rot) {
        const int pr = i >> 1;
        const float o = ldf<S>(dr + R + (i ^ 1));
        v = (i & 1) ? v * cs[pr] + o * cs[half + pr]
                    : v * cs[pr] - o * cs[half + pr];
      }
      stf<S>(kr + R + i, v);
    }
  }
  const int dq = dim + rd;
  for (int i = threadIdx.x; i < H * rd; i += 256) {
    const int h = i / rd, k = i % rd;
    const S* qr = q + (size_t)t * ldq + (size_t)h * dq + dim;
    float v = ldf<S>(qr + k);
    if (k < rot) {
      const int pr = k >> 1;
      const float o = ldf<S>(qr + (k ^ 1));
      v = (k & 1) ? v * cs[pr] + o * cs[half + pr]
                  : v * cs[pr] - o * cs[half + pr];
    }
    stf<S>(qf + ((size_t)t * H + h) * dkc + R + k, v);
  }
}

// out[t, h*dv + d] = o[h, t, d] * sigmoid(g[t, h*dv + d]): head-major
// per-head results back to token rows, times the output gate.
template <typename S, int V>
__global__ void __launch_bounds__(256) gate_heads_kernel(
    S* __restrict__ out, const S* __restrict__ o, const S* __restrict__ g,
    i64 ldg, int T, int H, int dv) {
  const int per = dv / V;
  const i64 total = (i64)T * H * per;
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (i64)gridDim.x * 256) {
    const int d = (int)(i % per) * V;
    const int h = (int)((i / per) % H);
    const i64 t = i / ((i64)per * H);
    float gv[4], ov[4];
    ldv<S, V>(g + t * ldg + (i64)h * dv + d, gv);
    ldv<S, V>(o + ((i64)h * T + t) * dv + d, ov);
#pragma unroll
    for (int j = 0; j < V; ++j) ov[j] = ov[j] / (1.0f + expf(-gv[j]));
    stv<S, V>(out + (t * H + h) * dv + d, ov);
  }
}

// out = max(z, 0)^2, rows of z at stride ldz.
template <typename S, int V>
__global__ void __launch_bounds__(256) relu2_kernel(
    S* __restrict__ out, const S* __restrict__ z, i64 ldz, int T, int F) {
  const i64 per = F / V;
  const i64 total = (i64)T * per;
  for (i64 i = (i64)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (i64)gridDim.x * 256) {
    const i64 t = i / per;
    const int c = (int)(i % per) * V;
    float v[4];
    ldv<S, V>(z + t * ldz + c, v);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float r = fmaxf(v[j], 0.f);
      v[j] = r * r;
    }
    stv<S, V>(out + t * F + c, v);
  }
}

inline bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

}  // namespace

AF_EXPORT int afm_embed_streams(void* x, const void* table, const void* ids,
                                int T, int ns, int W, int dt, void* stream) {
  if (T == 0) return 0;
  if (ns < 1) return 9003;
  hipStream_t s = (hipStream_t)stream;
  if (dt == 0)
    embed_streams_kernel<u16><<<T, 256, 0, s>>>((float*)x, (const u16*)table,
                                                (const i32*)ids, ns, W);
  else if (dt == 1)
    embed_streams_kernel<float><<<T, 256, 0, s>>>(
        (float*)x, (const float*)table, (const i32*)ids, ns, W);
  else
    return 9002;
  return af_last_err();
}

template <typename S>
static int launch_hyper_step(float* x, const void* y, i64 ldy,
                             const float* mixm, const float* outv,
                             const float* inv, const void* normw, float eps,
                             float* n, int T, int ns, int W, int norm_mode,
                             ConvTail ct, hipStream_t s) {
  const bool vec = W % 4 == 0 && ldy % 4 == 0 && al16(x) && al16(n) &&
                   al16(y) && al16(normw) && al16(ct.state) && al16(ct.h);
  // few rows of many columns: one column group per thread
  const bool wide = T <= 512 && W / (vec ? 4 : 1) > 256;
#define HS(MS, V)                                                            \
  do {                                                                       \
    if (wide)                                                                \
      hyper_step_kernel<S, MS, V, 1024><<<T, 1024, 0, s>>>(                  \
          x, (const S*)y, ldy, mixm, outv, inv, (const S*)normw, eps, n, ns, \
          W, norm_mode, ct);                                                 \
    else                                                                     \
      hyper_step_kernel<S, MS, V, 256><<<T, 256, 0, s>>>(                    \
          x, (const S*)y, ldy, mixm, outv, inv, (const S*)normw, eps, n, ns, \
          W, norm_mode, ct);                                                 \
  } while (0)
  if (ns <= 4) { if (vec) HS(4, 4); else HS(4, 1); }
  else if (ns <= 8) { if (vec) HS(8, 4); else HS(8, 1); }
  else { if (vec) HS(16, 4); else HS(16, 1); }
#undef HS
  return af_last_err();
}

// x [T, ns, W] fp32 in place; y [T, W] at row stride ldy (or null); mixm
// [ns, ns] indexed [from, to], outv / inv [ns] fp32; normw [W]; n [T, W] fp32.
// conv_w [W, taps] switches the convolution tail on (one row per sequence;
// needs the norm): conv_state [slots, max(taps-1, 1), W] fp32, sslot / pos
// [T], h [T, W] in the storage dtype.
AF_EXPORT int afm_hyper_step(void* x, const void* y, i64 ldy, const void* mixm,
                             const void* outv, const void* inv,
                             const void* normw, float eps, void* n, int T,
                             int ns, int W, int norm_mode, const void* conv_w,
                             void* conv_state, const void* sslot,
                             const void* pos, int taps, void* h, int dt,
                             void* stream) {
  if (T == 0) return 0;
  if (ns < 1 || ns > 16) return 9003;
  if (y && (!mixm || !outv)) return 9003;
  if (inv && (!n || (norm_mode == 1 && !normw))) return 9003;
  if (conv_w && (!inv || norm_mode != 1 || taps < 1 || !conv_state || !sslot ||
                 !pos || !h)) return 9003;
  const ConvTail ct{conv_w, (float*)conv_state, (const i32*)sslot,
                    (const i32*)pos, h, taps};
  hipStream_t s = (hipStream_t)stream;
  if (dt == 0)
    return launch_hyper_step<u16>((float*)x, y, ldy, (const float*)mixm,
        (const float*)outv, (const float*)inv, normw, eps, (float*)n, T, ns, W,
        norm_mode, ct, s);
  if (dt == 1)
    return launch_hyper_step<float>((float*)x, y, ldy, (const float*)mixm,
        (const float*)outv, (const float*)inv, normw, eps, (float*)n, T, ns, W,
        norm_mode, ct, s);
  return 9002;
}

// h [T, W] in the storage dtype; n [T, W] fp32; w [W, taps]; state [slots,
// max(taps-1, 1), W] fp32.  Runs the convolution, then moves the slots on.
AF_EXPORT int afm_canon_conv(void* h, const void* n, const void* w,
                             void* state, const void* row_seq, const void* cu,
                             const void* q_start, const void* sslot, int T,
                             int B, int W, int taps, int dt, void* stream) {
  if (T == 0) return 0;
  if (taps < 1) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = W % 4 == 0 && al16(h) && al16(n) && al16(state);
  dim3 grid((T + CONV_ROWS - 1) / CONV_ROWS,
            vec ? (W / 4 + 255) / 256 : (W + 255) / 256);
#define CC(S, V)                                                              \
  canon_conv_kernel<S, V><<<grid, 256, 0, s>>>(                               \
      (S*)h, (const float*)n, (const S*)w, (const float*)state,               \
      (const i32*)row_seq, (const i32*)cu, (const i32*)q_start,               \
      (const i32*)sslot, T, W, taps)
  if (dt == 0) { if (vec) CC(u16, 4); else CC(u16, 1); }
  else if (dt == 1) { if (vec) CC(float, 4); else CC(float, 1); }
  else return 9002;
#undef CC
  if (taps > 1)
    canon_state_kernel<<<dim3(B, (W + 255) / 256), 256, 0, s>>>(
        (float*)state, (const float*)n, (const i32*)cu, (const i32*)q_start,
        (const i32*)sslot, W, taps);
  return af_last_err();
}

AF_EXPORT int afm_latent_prep(void* qf, void* kc, const void* q, i64 ldq,
                              const void* dkv, i64 lddkv,
                              const void* normw, const void* inv_freq,
                              const void* positions, const void* slots,
                              float eps, int T, int H, int dim, int rd, int R,
                              int rot, int dt, void* stream) {
  if (T == 0) return 0;
  if (rot < 0 || rot > rd || (rot & 1) || (rot && !inv_freq)) return 9003;
  hipStream_t s = (hipStream_t)stream;
  const size_t sm = (size_t)(rot > 0 ? rot : 1) * sizeof(float);
  if (dt == 0)
    latent_prep_kernel<u16><<<T, 256, sm, s>>>(
        (u16*)qf, (u16*)kc, (const u16*)q, ldq, (const u16*)dkv, lddkv,
        (const u16*)normw, (const float*)inv_freq,
        (const i32*)positions, (const i64*)slots, eps, T, H, dim, rd, R, rot);
  else if (dt == 1)
    latent_prep_kernel<float><<<T, 256, sm, s>>>(
        (float*)qf, (float*)kc, (const float*)q, ldq, (const float*)dkv, lddkv,
        (const float*)normw, (const float*)inv_freq,
        (const i32*)positions, (const i64*)slots, eps, T, H, dim, rd, R, rot);
  else
    return 9002;
  return af_last_err();
}

AF_EXPORT int afm_gate_heads(void* out, const void* o, const void* g, i64 ldg,
                             int T, int H, int dv, int dt, void* stream) {
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = dv % 4 == 0 && ldg % 4 == 0 && al16(out) && al16(o) &&
                   al16(g);
  const i64 total = (i64)T * H * (vec ? dv / 4 : dv);
  const int grid = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
#define GH(S, V)                                                              \
  gate_heads_kernel<S, V><<<grid, 256, 0, s>>>((S*)out, (const S*)o,          \
                                               (const S*)g, ldg, T, H, dv)
  if (dt == 0) { if (vec) GH(u16, 4); else GH(u16, 1); }
  else if (dt == 1) { if (vec) GH(float, 4); else GH(float, 1); }
  else return 9002;
#undef GH
  return af_last_err();
}

AF_EXPORT int afm_relu2(void* out, const void* z, i64 ldz, int T, int F,
                        int dt, void* stream) {
  if (T == 0 || F == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool vec = F % 4 == 0 && ldz % 4 == 0 && al16(out) && al16(z);
  const i64 total = (i64)T * (vec ? F / 4 : F);
  const int grid = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
#define R2(S, V) relu2_kernel<S, V><<<grid, 256, 0, s>>>((S*)out, (const S*)z, ldz, T, F)
  if (dt == 0) { if (vec) R2(u16, 4); else R2(u16, 1); }
  else if (dt == 1) { if (vec) R2(float, 4); else R2(float, 1); }
  else return 9002;
#undef R2
  return af_last_err();
}
