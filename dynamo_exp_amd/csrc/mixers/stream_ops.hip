// Row-wise kernels of layer-listed (hybrid) models on gfx950: the multi-stream
// residual ("hyper-connections") update fused with the next sublayer's
// read-in and RMS norm, the embedding gather into fp32 streams, gated
// feed-forward activations, per-head q/k normalisation fused with the paged
// cache write, the two-map (differential) attention combine, and the
// single-residual step of parallel blocks (several sublayer outputs and a
// unit-RMS addend joined in one pass with the next RMS or layer norm).
//
// Every kernel is a template over the activation element (bf16 bits or
// float); reductions, norms, the residual streams and every scale are fp32
// whatever the element is.  Sizes are run-time arguments: nothing here is
// specialised for one model's widths.
#include "../kernels/common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaxStreams = 8;

template <typename T> __device__ __forceinline__ float ldf(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
template <> __device__ __forceinline__ float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <typename T> __device__ __forceinline__ void stf(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, int64_t i, float v) { p[i] = v; }

// V consecutive elements as floats (V = 4: one 8-byte / 16-byte access; V = 1: scalar)
template <typename T, int V> __device__ __forceinline__ void ldv(const T* p, float* o) {
  if constexpr (V == 1) {
    o[0] = ldf<T>(p, 0);
  } else if constexpr (sizeof(T) == 2) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    o[0] = bf16lo(w.x), o[1] = bf16hi(w.x), o[2] = bf16lo(w.y), o[3] = bf16hi(w.y);
  } else {
    const f32x4 w = *reinterpret_cast<const f32x4*>(p);
    o[0] = w[0], o[1] = w[1], o[2] = w[2], o[3] = w[3];
  }
}
template <typename T, int V> __device__ __forceinline__ void stv(T* p, const float* v) {
  if constexpr (V == 1) {
    stf<T>(p, 0, v[0]);
  } else if constexpr (sizeof(T) == 2) {
    uint2 w;
    w.x = pack_bf16x2(v[0], v[1]);
    w.y = pack_bf16x2(v[2], v[3]);
    *reinterpret_cast<uint2*>(p) = w;
  } else {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
  }
}

template <typename T, int V> __device__ __forceinline__ void cpv(T* dst, const T* src) {  // raw copy of V elements
  if constexpr (V == 1) {
    dst[0] = src[0];
  } else if constexpr (sizeof(T) == 2) {
    *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(src);
  } else {
    *reinterpret_cast<f32x4*>(dst) = *reinterpret_cast<const f32x4*>(src);
  }
}

// One residual step of a model with S parallel residual streams X [rows, S, W]
// (fp32, updated in place).  With y (the previous sublayer's output):
//     X_t <- sum_s mix[s, t] X_s + gain[t] * y          for every stream t
// then, with read-in weights rin [S]:  u = sum_s rin[s] X_s  and
//     out = u / sqrt(mean(u^2) + eps) * nw              (nw fp32 [W]; nw == null: out = u)
// S = 1, mix = [1], gain = [1], rin = [1] is the ordinary pre-norm residual.
template <typename T, int V>
__global__ void __launch_bounds__(kThreads) stream_step_kernel(float* __restrict__ X, const T* __restrict__ y,
                                                               int64_t y_stride, const float* __restrict__ mix,
                                                               const float* __restrict__ gain,
                                                               const float* __restrict__ rin,
                                                               const float* __restrict__ nw, float eps,
                                                               T* __restrict__ out, int64_t out_stride, int S, int W) {
  __shared__ float red[16];
  __shared__ float sm[kMaxStreams * kMaxStreams + 2 * kMaxStreams];
  const int64_t row = blockIdx.x;
  float* x = X + row * (int64_t)S * W;
  float* s_mix = sm;
  float* s_gain = sm + kMaxStreams * kMaxStreams;
  float* s_in = s_gain + kMaxStreams;
  if (threadIdx.x < S * S && y) s_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    s_gain[threadIdx.x] = y ? gain[threadIdx.x] : 0.f;
    s_in[threadIdx.x] = rin ? rin[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float ss = 0.f;
  for (int c = threadIdx.x * V; c < W; c += kThreads * V) {
    float v[kMaxStreams][V];
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s)
      if (s < S) ldv<float, V>(x + (int64_t)s * W + c, v[s]);
    if (y) {
      float yv[V], n[kMaxStreams][V];
      ldv<T, V>(y + row * y_stride + c, yv);
#pragma unroll
      for (int t = 0; t < kMaxStreams; ++t) {
        if (t < S) {
#pragma unroll
          for (int e = 0; e < V; ++e) {
            float a = s_gain[t] * yv[e];
#pragma unroll
            for (int s = 0; s < kMaxStreams; ++s)
              if (s < S) a += s_mix[s * S + t] * v[s][e];
            n[t][e] = a;
          }
          stv<float, V>(x + (int64_t)t * W + c, n[t]);
        }
      }
#pragma unroll
      for (int t = 0; t < kMaxStreams; ++t)
        if (t < S) {
#pragma unroll
          for (int e = 0; e < V; ++e) v[t][e] = n[t][e];
        }
    }
    if (rin) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        float uu = 0.f;
#pragma unroll
        for (int s = 0; s < kMaxStreams; ++s)
          if (s < S) uu += s_in[s] * v[s][e];
        ss += uu * uu;
      }
    }
  }
  if (!rin) return;
  const float tot = block_reduce_sum(ss, red);
  const float r = nw ? rsqrtf(tot / (float)W + eps) : 1.f;
  // second pass: this thread re-reads the stream values it wrote itself
  for (int c = threadIdx.x * V; c < W; c += kThreads * V) {
    float u[V], o[V], xv[V], wv[V];
#pragma unroll
    for (int e = 0; e < V; ++e) u[e] = 0.f;
    for (int s = 0; s < S; ++s) {
      ldv<float, V>(x + (int64_t)s * W + c, xv);
#pragma unroll
      for (int e = 0; e < V; ++e) u[e] += s_in[s] * xv[e];
    }
    if (nw) ldv<float, V>(nw + c, wv);
#pragma unroll
    for (int e = 0; e < V; ++e) o[e] = nw ? u[e] * r * wv[e] : u[e];
    stv<T, V>(out + row * out_stride + c, o);
  }
}

// X[t, s, :] = table[ids[t], :] * scale (+ ptab[pos[t], :], a learned vector per position)
// for every stream s (fp32 streams; product and sum are fp32)
template <typename T>
__global__ void __launch_bounds__(kThreads) embed_streams_kernel(float* __restrict__ X, const T* __restrict__ table,
                                                                 const int64_t* __restrict__ ids, int S, int W,
                                                                 int64_t vocab, const T* __restrict__ ptab,
                                                                 const int64_t* __restrict__ pos, int64_t n_pos,
                                                                 float scale) {
  const int64_t t = blockIdx.x;
  const int64_t id = ids[t];
  const bool ok = id >= 0 && id < vocab;
  const int64_t p = ptab ? pos[t] : -1;
  const bool pok = p >= 0 && p < n_pos;
  for (int c = threadIdx.x; c < W; c += kThreads) {
    float v = ok ? ldf<T>(table, id * (int64_t)W + c) * scale : 0.f;
    if (pok) v += ldf<T>(ptab, p * (int64_t)W + c);
    for (int s = 0; s < S; ++s) X[(t * S + s) * (int64_t)W + c] = v;
  }
}

// out[t, :] = table[ids[t], :] (zeros for ids outside the table)
template <typename T>
__global__ void __launch_bounds__(kThreads) gather_rows_kernel(T* __restrict__ out, const T* __restrict__ table,
                                                               const int64_t* __restrict__ ids, int W, int64_t vocab) {
  const int64_t t = blockIdx.x;
  const int64_t id = ids[t];
  const bool ok = id >= 0 && id < vocab;
  for (int c = threadIdx.x; c < W; c += kThreads) out[t * (int64_t)W + c] = ok ? table[id * (int64_t)W + c] : (T)0;
}

// One step of a single fp32 residual x [rows, W], in place:
//     x <- x + a + b + c / sqrt(mean(c^2) + eps) * cw        (a, b, c optional)
// then  xc = x in T (when xc), and the norm that follows (when out):
//     norm 1 (RMS):    out = x / sqrt(mean(x^2) + eps) * nw
//     norm 2 (layer):  out = (x - mean) / sqrt(mean((x - mean)^2) + eps) * nw + nb
// The row stays in registers between the passes (W <= kThreads * V * kResChunks)
// or is re-read from x by the thread that wrote it.
constexpr int kResChunks = 8;
template <typename T, int V>
__global__ void __launch_bounds__(kThreads) residual_step_kernel(
    float* __restrict__ X, const T* __restrict__ a, int64_t a_stride, const T* __restrict__ b, int64_t b_stride,
    const T* __restrict__ c, int64_t c_stride, const float* __restrict__ cw, const T* __restrict__ cg,
    int64_t cg_stride, const float* __restrict__ cgb, float eps, int norm, const float* __restrict__ nw,
    const float* __restrict__ nb, T* __restrict__ out, T* __restrict__ xc, int W) {
  __shared__ float red[16];
  const int64_t row = blockIdx.x;
  float* x = X + row * (int64_t)W;
  float rc = 0.f;
  // the addend c at columns e .. e + V - 1, gated by sigmoid(cg + cgb) when a gate is given
  auto load_c = [&](int e, float* v) {
    ldv<T, V>(c + row * c_stride + e, v);
    if (cg) {
      float gt[V], gb[V];
      ldv<T, V>(cg + row * cg_stride + e, gt);
      if (cgb) ldv<float, V>(cgb + e, gb);
#pragma unroll
      for (int i = 0; i < V; ++i) v[i] *= 1.f / (1.f + expf(-(gt[i] + (cgb ? gb[i] : 0.f))));
    }
  };
  // (gated) addend: its chunks stay in registers between the mean square and the sum
  float cv[kResChunks][V];
  if (c) {
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < kResChunks; ++k) {
      const int e = (threadIdx.x + k * kThreads) * V;
      if (e < W) {
        load_c(e, cv[k]);
#pragma unroll
        for (int i = 0; i < V; ++i) ss += cv[k][i] * cv[k][i];
      }
    }
    for (int e = (threadIdx.x + kResChunks * kThreads) * V; e < W; e += kThreads * V) {
      float v[V];
      load_c(e, v);
#pragma unroll
      for (int i = 0; i < V; ++i) ss += v[i] * v[i];
    }
    rc = rsqrtf(block_reduce_sum(ss, red) / (float)W + eps);
    __syncthreads();
  }
  const bool keep = W <= kThreads * V * kResChunks;
  float r[kResChunks][V];
  float sum = 0.f;
  const bool touch = a || b || c;
#pragma unroll
  for (int k = 0; k < kResChunks; ++k) {
    const int e = (threadIdx.x + k * kThreads) * V;
    if (e < W) {
      ldv<float, V>(x + e, r[k]);
      float t[V];
      if (a) {
        ldv<T, V>(a + row * a_stride + e, t);
#pragma unroll
        for (int i = 0; i < V; ++i) r[k][i] += t[i];
      }
      if (b) {
        ldv<T, V>(b + row * b_stride + e, t);
#pragma unroll
        for (int i = 0; i < V; ++i) r[k][i] += t[i];
      }
      if (c) {
        float w[V];
        ldv<float, V>(cw + e, w);
#pragma unroll
        for (int i = 0; i < V; ++i) r[k][i] += cv[k][i] * rc * w[i];
      }
      if (touch) stv<float, V>(x + e, r[k]);
      if (xc) stv<T, V>(xc + row * (int64_t)W + e, r[k]);
#pragma unroll
      for (int i = 0; i < V; ++i) sum += r[k][i];
    }
  }
  if (!keep) {  // wide rows: the same arithmetic, chunk by chunk through x
    for (int e = (threadIdx.x + kResChunks * kThreads) * V; e < W; e += kThreads * V) {
      float v[V], t[V];
      ldv<float, V>(x + e, v);
      if (a) {
        ldv<T, V>(a + row * a_stride + e, t);
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] += t[i];
      }
      if (b) {
        ldv<T, V>(b + row * b_stride + e, t);
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] += t[i];
      }
      if (c) {
        float w[V];
        load_c(e, t);
        ldv<float, V>(cw + e, w);
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] += t[i] * rc * w[i];
      }
      if (touch) stv<float, V>(x + e, v);
      if (xc) stv<T, V>(xc + row * (int64_t)W + e, v);
#pragma unroll
      for (int i = 0; i < V; ++i) sum += v[i];
    }
  }
  if (!norm) return;
  float mean = 0.f;
  if (norm == 2) {
    mean = block_reduce_sum(sum, red) / (float)W;
    __syncthreads();
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < kResChunks; ++k) {
    const int e = (threadIdx.x + k * kThreads) * V;
    if (e < W) {
#pragma unroll
      for (int i = 0; i < V; ++i) ss += (r[k][i] - mean) * (r[k][i] - mean);
    }
  }
  if (!keep) {
    for (int e = (threadIdx.x + kResChunks * kThreads) * V; e < W; e += kThreads * V) {
      float v[V];
      ldv<float, V>(x + e, v);
#pragma unroll
      for (int i = 0; i < V; ++i) ss += (v[i] - mean) * (v[i] - mean);
    }
  }
  const float rs = rsqrtf(block_reduce_sum(ss, red) / (float)W + eps);
#pragma unroll
  for (int k = 0; k < kResChunks; ++k) {
    const int e = (threadIdx.x + k * kThreads) * V;
    if (e < W) {
      float w[V], bb[V], o[V];
      ldv<float, V>(nw + e, w);
      if (norm == 2) ldv<float, V>(nb + e, bb);
#pragma unroll
      for (int i = 0; i < V; ++i) o[i] = (r[k][i] - mean) * rs * w[i] + (norm == 2 ? bb[i] : 0.f);
      stv<T, V>(out + row * (int64_t)W + e, o);
    }
  }
  if (!keep) {
    for (int e = (threadIdx.x + kResChunks * kThreads) * V; e < W; e += kThreads * V) {
      float v[V], w[V], bb[V], o[V];
      ldv<float, V>(x + e, v);
      ldv<float, V>(nw + e, w);
      if (norm == 2) ldv<float, V>(nb + e, bb);
#pragma unroll
      for (int i = 0; i < V; ++i) o[i] = (v[i] - mean) * rs * w[i] + (norm == 2 ? bb[i] : 0.f);
      stv<T, V>(out + row * (int64_t)W + e, o);
    }
  }
}

// Weighted sum over the results of all layers so far (a depth average):
//     dst[r, :] = sum_{j < n} w[j] * stack[j][row(r), :]        row(r) = rows ? rows[r] : r
// stack [>= n, T, W] fp32, one [T, W] plane per layer result; dst fp32 [n_rows, W] (it may be a
// later plane of the same stack); then, when out: out = dst / sqrt(mean(dst^2) + eps) * nw in T
// (nw one weight per column).  With c (the last sublayer's output, [T, c_stride] in T) the newest
// plane n - 1 first takes its closing addend, plane <- plane + c / sqrt(mean(c^2) + eps) * cw, and
// is written back (without `rows`; with them the sum alone uses it, a row may be listed twice).
// Sums in the order j = 0, 1, ..., all fp32.  The row stays in registers between the sum and the
// norm (W <= kThreads * V * kResChunks) or is re-read from dst.
template <typename T, int V>
__global__ void __launch_bounds__(kThreads) depth_mix_kernel(float* __restrict__ dst, float* __restrict__ stack,
                                                             int64_t plane, int n, const float* __restrict__ w,
                                                             const int64_t* __restrict__ rows, float eps,
                                                             const float* __restrict__ nw, T* __restrict__ out,
                                                             const T* __restrict__ c, int64_t c_stride,
                                                             const float* __restrict__ cw, int W) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t row = rows ? rows[r] : r;
  float* src = stack + row * (int64_t)W;
  float* x = dst + r * (int64_t)W;
  float rc = 0.f;
  if (c) {
    float cs = 0.f;
    for (int e = threadIdx.x * V; e < W; e += kThreads * V) {
      float t[V];
      ldv<T, V>(c + row * c_stride + e, t);
#pragma unroll
      for (int i = 0; i < V; ++i) cs += t[i] * t[i];
    }
    rc = rsqrtf(block_reduce_sum(cs, red) / (float)W + eps);
    __syncthreads();
  }
  // the weighted sum of columns e .. e + V - 1 over the planes
  auto mix = [&](int e, float* a) {
#pragma unroll
    for (int i = 0; i < V; ++i) a[i] = 0.f;
    for (int j = 0; j < n; ++j) {
      float t[V];
      ldv<float, V>(src + j * plane + e, t);
      if (c && j == n - 1) {
        float cv[V], g[V];
        ldv<T, V>(c + row * c_stride + e, cv);
        ldv<float, V>(cw + e, g);
#pragma unroll
        for (int i = 0; i < V; ++i) t[i] += cv[i] * rc * g[i];
        if (!rows) stv<float, V>(src + j * plane + e, t);
      }
      const float wj = w[j];
#pragma unroll
      for (int i = 0; i < V; ++i) a[i] += wj * t[i];
    }
  };
  float acc[kResChunks][V];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < kResChunks; ++k) {
    const int e = (threadIdx.x + k * kThreads) * V;
    if (e < W) {
      mix(e, acc[k]);
      stv<float, V>(x + e, acc[k]);
#pragma unroll
      for (int i = 0; i < V; ++i) ss += acc[k][i] * acc[k][i];
    }
  }
  for (int e = (threadIdx.x + kResChunks * kThreads) * V; e < W; e += kThreads * V) {
    float a[V];
    mix(e, a);
    stv<float, V>(x + e, a);
#pragma unroll
    for (int i = 0; i < V; ++i) ss += a[i] * a[i];
  }
  if (!out) return;
  const float rs = rsqrtf(block_reduce_sum(ss, red) / (float)W + eps);
#pragma unroll
  for (int k = 0; k < kResChunks; ++k) {
    const int e = (threadIdx.x + k * kThreads) * V;
    if (e < W) {
      float g[V], o[V];
      ldv<float, V>(nw + e, g);
#pragma unroll
      for (int i = 0; i < V; ++i) o[i] = acc[k][i] * rs * g[i];
      stv<T, V>(out + r * (int64_t)W + e, o);
    }
  }
  for (int e = (threadIdx.x + kResChunks * kThreads) * V; e < W; e += kThreads * V) {
    float a[V], g[V], o[V];
    ldv<float, V>(x + e, a);  // written by this thread above
    ldv<float, V>(nw + e, g);
#pragma unroll
    for (int i = 0; i < V; ++i) o[i] = a[i] * rs * g[i];
    stv<T, V>(out + r * (int64_t)W + e, o);
  }
}

// out [rows, n] = x / sqrt(mean(x^2) + eps) * w over a column section x [rows, n] of wider rows
// (a low-rank latent between its two projections): one wave per row, fp32 sums
template <typename T>
__global__ void __launch_bounds__(kThreads) section_norm_kernel(T* __restrict__ out, const T* __restrict__ x,
                                                                int64_t x_stride, const float* __restrict__ w,
                                                                int rows, int n, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * x_stride;
  float ss = 0.f;
  for (int e = lane; e < n; e += 64) {
    const float v = ldf<T>(xr, e);
    ss += v * v;
  }
  const float rs = rsqrtf(wave_reduce_sum(ss) / (float)n + eps);
  for (int e = lane; e < n; e += 64) stf<T>(out, row * n + e, ldf<T>(xr, e) * rs * (w ? w[e] : 1.f));
}

__device__ __forceinline__ float act_fn(float z, int act) {
  if (act == 5) return tanhf(z);
  if (act == 0) return fmaxf(z, 0.f);           // relu
  if (act == 1) return z / (1.f + __expf(-z));  // silu
  if (act == 3) return 1.f / (1.f + __expf(-z));  // sigmoid
  if (act == 4) {                                 // relu squared
    const float r = fmaxf(z, 0.f);
    return r * r;
  }
  const float c = 0.7978845608028654f;          // gelu, tanh form
  return 0.5f * z * (1.f + tanhf(c * (z + 0.044715f * z * z * z)));
}

// out [rows, F] = act(gate) * up  (up null: act(gate)); gate and up are column
// sections of wider rows (a gated feed-forward's [gate | up], an output gate
// that is part of a fused projection)
template <typename T, int V>
__global__ void __launch_bounds__(kThreads) act_mul_kernel(T* __restrict__ out, const T* __restrict__ gate,
                                                           int64_t g_stride, const T* __restrict__ up,
                                                           int64_t u_stride, int F, int64_t out_stride, int act,
                                                           float limit, float alpha) {
  const int64_t r = blockIdx.y;
  for (int c = (blockIdx.x * kThreads + threadIdx.x) * V; c < F; c += gridDim.x * kThreads * V) {
    float g[V], u[V], o[V];
    ldv<T, V>(gate + r * g_stride + c, g);
    if (up) ldv<T, V>(up + r * u_stride + c, u);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      if (act == 6) {  // clamped gated unit: g sigmoid(alpha g) (u + 1), g <= limit, |u| <= limit
        const float gc = fminf(g[e], limit), uc = fminf(fmaxf(u[e], -limit), limit);
        o[e] = gc / (1.f + __expf(-alpha * gc)) * (uc + 1.f);
      } else {
        o[e] = act_fn(g[e], act) * (up ? u[e] : 1.f);
      }
    }
    stv<T, V>(out + r * out_stride + c, o);
  }
}

// Per token row of a fused projection output x = [q | k | v]:
//   q: n_q vectors of d; with qw: unit RMS times qw [d]; with temp_coef != 0 a
//      position-dependent gain 1 + coef * ln(floor((p + 1) / every) + 1); in place
//   k: n_k vectors of d at column k_off; with kw: unit RMS times kw; written to
//      the K cache row of the token's slot (kc [slots, n_k * d])
//   v: v_mode 0: no V cache (V is the K cache); 1: the k section as projected
//      (before its norm) is the value; 2: v_w columns at v_off are the value,
//      mixed with an earlier layer's values of the same token when v_first is
//      given: (1 - v_lambda) v + v_lambda v_first, in fp32
// slot < 0: nothing is cached for the row.
template <typename T, int V>
__global__ void __launch_bounds__(kThreads) headprep_cache_kernel(
    T* __restrict__ x, int64_t x_stride, const int64_t* __restrict__ pos, const int64_t* __restrict__ slots,
    int n_q, int n_k, int d, int k_off, const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    float temp_coef, double temp_every, T* __restrict__ kc, T* __restrict__ vc, int v_mode, int v_off, int v_w,
    const T* __restrict__ v_first, int64_t vf_stride, float v_lambda, int lpv) {
  // lpv lanes (a power of two) share one head vector, so a wave works on 64 / lpv
  // vectors at once and their loads overlap; the sum of squares is reduced inside the group
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = kThreads / 64;
  const int per_wave = 64 / lpv, grp = lane / lpv, gl = lane - grp * lpv;
  T* row = x + t * x_stride;
  const int64_t slot = slots[t];
  const int k_w = n_k * d;
  float gain = 1.f;
  if (temp_coef != 0.f) {
    const double k = floor((double)(pos[t] + 1) / temp_every);
    gain = 1.f + temp_coef * logf((float)k + 1.f);
  }
  const bool q_work = qw != nullptr || temp_coef != 0.f;
  for (int v = wid * per_wave + grp; v < n_q + n_k; v += nw * per_wave) {
    const bool is_q = v < n_q;
    if (is_q && !q_work) continue;
    if (!is_q && slot < 0) continue;
    T* src = is_q ? row + (int64_t)v * d : row + k_off + (int64_t)(v - n_q) * d;
    const float* w = is_q ? qw : kw;
    float r = 1.f;
    if (w) {
      float ss = 0.f;
      for (int e = gl * V; e < d; e += lpv * V) {
        float a[V];
        ldv<T, V>(src + e, a);
#pragma unroll
        for (int i = 0; i < V; ++i) ss += a[i] * a[i];
      }
      for (int o = lpv >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
      r = rsqrtf(ss / (float)d + eps);
    }
    T* kd = is_q ? src : kc + slot * (int64_t)k_w + (int64_t)(v - n_q) * d;
    T* vd = (!is_q && v_mode == 1) ? vc + slot * (int64_t)k_w + (int64_t)(v - n_q) * d : nullptr;
    const float g = is_q ? gain : 1.f;
    for (int e = gl * V; e < d; e += lpv * V) {
      float a[V], wv[V];
      ldv<T, V>(src + e, a);
      if (vd) cpv<T, V>(vd + e, src + e);
      if (w) ldv<float, V>(w + e, wv);
#pragma unroll
      for (int i = 0; i < V; ++i) a[i] = a[i] * (w ? r * wv[i] : 1.f) * g;
      stv<T, V>(kd + e, a);
    }
  }
  if (v_mode == 2 && slot >= 0) {
    const T* vs = row + v_off;
    T* vd = vc + slot * (int64_t)v_w;
    if (v_first) {
      const T* vf = v_first + t * vf_stride;
      for (int e = threadIdx.x * V; e < v_w; e += kThreads * V) {
        float a[V], f[V];
        ldv<T, V>(vs + e, a);
        ldv<T, V>(vf + e, f);
#pragma unroll
        for (int i = 0; i < V; ++i) a[i] = (1.f - v_lambda) * a[i] + v_lambda * f[i];
        stv<T, V>(vd + e, a);
      }
    } else {
      for (int e = threadIdx.x * V; e < v_w; e += kThreads * V) cpv<T, V>(vd + e, vs + e);
    }
  }
}

// Two-map attention combine: a [rows, H, 2, dv] fp32 (map outputs over the
// same values)  ->  out [rows, H, dv] = unit_rms(a1 - lam * a2) * post, times
// sigmoid(gate[row, head]) when gate (logits [rows, gate_stride], one per head) is given.
// One wave per (row, head).
template <typename T>
__global__ void __launch_bounds__(kThreads) diff_combine_kernel(T* __restrict__ out, const float* __restrict__ a,
                                                                int64_t n_vec, int dv, float lam, float post,
                                                                float eps, const T* __restrict__ gate,
                                                                int64_t gate_stride, int H) {
  const int lane = threadIdx.x & 63;
  const int64_t v = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  if (v >= n_vec) return;
  const float* a1 = a + v * 2 * (int64_t)dv;
  const float* a2 = a1 + dv;
  float ss = 0.f;
  for (int e = lane; e < dv; e += 64) {
    const float o = a1[e] - lam * a2[e];
    ss += o * o;
  }
  float r = rsqrtf(wave_reduce_sum(ss) / (float)dv + eps) * post;
  if (gate) r /= 1.f + expf(-ldf<T>(gate, v / H * gate_stride + v % H));
  for (int e = lane; e < dv; e += 64) stf<T>(out, v * dv + e, (a1[e] - lam * a2[e]) * r);
}

}  // namespace

#define DISPATCH_T(f32, ...)          \
  if (f32) {                          \
    using T = float;                  \
    __VA_ARGS__;                      \
  } else {                            \
    using T = bf16_t;                 \
    __VA_ARGS__;                      \
  }

extern "C" {

int dxm_stream_step(float* X, const void* y, int64_t y_stride, const float* mix, const float* gain, const float* rin,
                    const float* nw, float eps, void* out, int64_t out_stride, int rows, int S, int W, int f32,
                    hipStream_t st) {
  if (S < 1 || S > kMaxStreams || W < 1) return 1;
  if (rows <= 0) return 0;
  if (y && (!mix || !gain)) return 2;
  if (rin && !out) return 3;
  const int esz = f32 ? 4 : 2;
  const bool vec = W % 4 == 0 && y_stride % 4 == 0 && out_stride % 4 == 0 && (uintptr_t)X % 16 == 0 &&
                   (uintptr_t)y % (4 * esz) == 0 && (uintptr_t)out % (4 * esz) == 0 && (uintptr_t)nw % 16 == 0;
  if (vec) {
    DISPATCH_T(f32, hipLaunchKernelGGL((stream_step_kernel<T, 4>), dim3(rows), dim3(kThreads), 0, st, X, (const T*)y,
                                       y_stride, mix, gain, rin, nw, eps, (T*)out, out_stride, S, W));
  } else {
    DISPATCH_T(f32, hipLaunchKernelGGL((stream_step_kernel<T, 1>), dim3(rows), dim3(kThreads), 0, st, X, (const T*)y,
                                       y_stride, mix, gain, rin, nw, eps, (T*)out, out_stride, S, W));
  }
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_embed_streams(float* X, const void* table, const int64_t* ids, int rows, int S, int W, int64_t vocab,
                      const void* ptab, const int64_t* pos, int64_t n_pos, float scale, int f32, hipStream_t st) {
  if (rows <= 0) return 0;
  if (ptab && !pos) return 1;
  DISPATCH_T(f32, hipLaunchKernelGGL(embed_streams_kernel<T>, dim3(rows), dim3(kThreads), 0, st, X, (const T*)table,
                                     ids, S, W, vocab, (const T*)ptab, pos, n_pos, scale));
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_gather_rows(void* out, const void* table, const int64_t* ids, int rows, int W, int64_t vocab, int f32,
                    hipStream_t st) {
  if (rows <= 0) return 0;
  DISPATCH_T(f32, hipLaunchKernelGGL(gather_rows_kernel<T>, dim3(rows), dim3(kThreads), 0, st, (T*)out,
                                     (const T*)table, ids, W, vocab));
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_residual_step(float* X, const void* a, int64_t a_stride, const void* b, int64_t b_stride, const void* c,
                      int64_t c_stride, const float* cw, const void* cg, int64_t cg_stride, const float* cgb, float eps,
                      int norm, const float* nw, const float* nb, void* out, void* xc, int rows, int W, int f32,
                      hipStream_t st) {
  if (rows <= 0) return 0;
  if (W < 1 || norm < 0 || norm > 2) return 1;
  if ((c && !cw) || (norm && (!nw || !out)) || (norm == 2 && !nb) || (cg && !c)) return 2;
  const int esz = f32 ? 4 : 2;
  auto al = [&](const void* p, int by) { return (uintptr_t)p % by == 0; };
  const bool vec = W % 4 == 0 && a_stride % 4 == 0 && b_stride % 4 == 0 && c_stride % 4 == 0 && cg_stride % 4 == 0 &&
                   al(X, 16) && al(a, 4 * esz) && al(b, 4 * esz) && al(c, 4 * esz) && al(cg, 4 * esz) && al(cgb, 16) &&
                   al(cw, 16) && al(nw, 16) && al(nb, 16) &&
                   al(out, 4 * esz) && al(xc, 4 * esz);
  if (vec) {
    DISPATCH_T(f32, hipLaunchKernelGGL((residual_step_kernel<T, 4>), dim3(rows), dim3(kThreads), 0, st, X, (const T*)a,
                                       a_stride, (const T*)b, b_stride, (const T*)c, c_stride, cw, (const T*)cg, cg_stride, cgb, eps,
                                       norm, nw, nb,
                                       (T*)out, (T*)xc, W));
  } else {
    DISPATCH_T(f32, hipLaunchKernelGGL((residual_step_kernel<T, 1>), dim3(rows), dim3(kThreads), 0, st, X, (const T*)a,
                                       a_stride, (const T*)b, b_stride, (const T*)c, c_stride, cw, (const T*)cg, cg_stride, cgb, eps,
                                       norm, nw, nb,
                                       (T*)out, (T*)xc, W));
  }
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_act_mul(void* out, const void* gate, int64_t g_stride, const void* up, int64_t u_stride, int rows, int F,
                int64_t out_stride, int act, float limit, float alpha, int f32, hipStream_t st) {
  if (rows <= 0 || F <= 0) return 0;
  if (act < 0 || act > 6 || (act == 6 && (!up || !(limit > 0.f)))) return 1;
  const int esz = f32 ? 4 : 2;
  const bool vec = F % 4 == 0 && g_stride % 4 == 0 && u_stride % 4 == 0 && out_stride % 4 == 0 &&
                   (uintptr_t)gate % (4 * esz) == 0 && (uintptr_t)up % (4 * esz) == 0 &&
                   (uintptr_t)out % (4 * esz) == 0;
  const int per = kThreads * (vec ? 4 : 1);
  const int gx = (F + per - 1) / per;
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    if (vec) {
      DISPATCH_T(f32, hipLaunchKernelGGL((act_mul_kernel<T, 4>), dim3(gx, nr), dim3(kThreads), 0, st,
                                         (T*)out + r0 * out_stride, (const T*)gate + r0 * g_stride, g_stride,
                                         up ? (const T*)up + r0 * u_stride : nullptr, u_stride, F, out_stride, act,
                                         limit, alpha));
    } else {
      DISPATCH_T(f32, hipLaunchKernelGGL((act_mul_kernel<T, 1>), dim3(gx, nr), dim3(kThreads), 0, st,
                                         (T*)out + r0 * out_stride, (const T*)gate + r0 * g_stride, g_stride,
                                         up ? (const T*)up + r0 * u_stride : nullptr, u_stride, F, out_stride, act,
                                         limit, alpha));
    }
  }
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_headprep_cache(void* x, int64_t x_stride, const int64_t* pos, const int64_t* slots, int rows, int n_q, int n_k,
                       int d, int k_off, const float* qw, const float* kw, float eps, float temp_coef,
                       double temp_every, void* kc, void* vc, int v_mode, int v_off, int v_w, const void* v_first,
                       int64_t vf_stride, float v_lambda, int f32, hipStream_t st) {
  if (rows <= 0) return 0;
  if (n_q < 0 || n_k < 0 || d < 1 || v_mode < 0 || v_mode > 2) return 1;
  if (n_k > 0 && !kc) return 2;
  if (v_mode != 0 && !vc) return 3;
  if (temp_coef != 0.f && !(temp_every > 0)) return 4;
  if (v_first && v_mode != 2) return 5;
  const int esz = f32 ? 4 : 2;
  const bool vec = d % 4 == 0 && k_off % 4 == 0 && x_stride % 4 == 0 && v_off % 4 == 0 && v_w % 4 == 0 &&
                   vf_stride % 4 == 0 && (uintptr_t)v_first % (4 * esz) == 0 &&
                   (uintptr_t)x % (4 * esz) == 0 && (uintptr_t)kc % (4 * esz) == 0 && (uintptr_t)vc % (4 * esz) == 0 &&
                   (uintptr_t)qw % 16 == 0 && (uintptr_t)kw % 16 == 0;
  // lanes per head vector: about two chunks of V elements per lane
  const int chunks = (d + (vec ? 4 : 1) - 1) / (vec ? 4 : 1);
  int lpv = 1;
  while (lpv < 64 && lpv * 2 < chunks) lpv <<= 1;
  if (vec) {
    DISPATCH_T(f32, hipLaunchKernelGGL((headprep_cache_kernel<T, 4>), dim3(rows), dim3(kThreads), 0, st, (T*)x,
                                       x_stride, pos, slots, n_q, n_k, d, k_off, qw, kw, eps, temp_coef, temp_every,
                                       (T*)kc, (T*)vc, v_mode, v_off, v_w, (const T*)v_first, vf_stride, v_lambda,
                                       lpv));
  } else {
    DISPATCH_T(f32, hipLaunchKernelGGL((headprep_cache_kernel<T, 1>), dim3(rows), dim3(kThreads), 0, st, (T*)x,
                                       x_stride, pos, slots, n_q, n_k, d, k_off, qw, kw, eps, temp_coef, temp_every,
                                       (T*)kc, (T*)vc, v_mode, v_off, v_w, (const T*)v_first, vf_stride, v_lambda,
                                       lpv));
  }
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_depth_mix(float* dst, float* stack, int64_t plane, int n, const float* w, const int64_t* rows, int n_rows,
                  float eps, const float* nw, void* out, const void* c, int64_t c_stride, const float* cw, int W,
                  int f32, hipStream_t st) {
  if (n_rows <= 0) return 0;
  if (n < 1 || W < 1 || !dst || !stack || !w || (out && !nw) || (c && !cw)) return 1;
  const int esz = f32 ? 4 : 2;
  auto al = [&](const void* p, int by) { return (uintptr_t)p % by == 0; };
  const bool vec = W % 4 == 0 && plane % 4 == 0 && c_stride % 4 == 0 && al(dst, 16) && al(stack, 16) && al(nw, 16) &&
                   al(out, 4 * esz) && al(c, 4 * esz) && al(cw, 16);
  if (vec) {
    DISPATCH_T(f32, hipLaunchKernelGGL((depth_mix_kernel<T, 4>), dim3(n_rows), dim3(kThreads), 0, st, dst, stack, plane,
                                       n, w, rows, eps, nw, (T*)out, (const T*)c, c_stride, cw, W));
  } else {
    DISPATCH_T(f32, hipLaunchKernelGGL((depth_mix_kernel<T, 1>), dim3(n_rows), dim3(kThreads), 0, st, dst, stack, plane,
                                       n, w, rows, eps, nw, (T*)out, (const T*)c, c_stride, cw, W));
  }
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_section_norm(void* out, const void* x, int64_t x_stride, const float* w, int rows, int n, float eps, int f32,
                     hipStream_t st) {
  if (rows <= 0) return 0;
  if (n < 1 || !out || !x) return 1;
  const int blocks = (rows + kThreads / 64 - 1) / (kThreads / 64);
  DISPATCH_T(f32, hipLaunchKernelGGL(section_norm_kernel<T>, dim3(blocks), dim3(kThreads), 0, st, (T*)out, (const T*)x,
                                     x_stride, w, rows, n, eps));
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_diff_combine(void* out, const float* a, int64_t n_vec, int dv, float lam, float post, float eps,
                     const void* gate, int64_t gate_stride, int H, int f32, hipStream_t st) {
  if (n_vec <= 0) return 0;
  if (gate && (H < 1 || n_vec % H)) return 1;
  const int64_t blocks = (n_vec + kThreads / 64 - 1) / (kThreads / 64);
  DISPATCH_T(f32, hipLaunchKernelGGL(diff_combine_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, st, (T*)out, a,
                                     n_vec, dv, lam, post, eps, (const T*)gate, gate_stride, H > 0 ? H : 1));
  DX_CHECK_LAUNCH();
  return 0;
}

}  // extern "C"
