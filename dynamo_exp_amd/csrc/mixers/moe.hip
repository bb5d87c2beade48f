// Mixture-of-experts kernels for gfx950: expert choice from router logits, the
// per-step plan (slots sorted by expert, on the device), grouped GEMMs over
// each expert's rows on the matrix cores, and the weighted combine.
//
// A step of T tokens with `top` experts each has R = T * top slots; slot
// t * top + k is token t's k-th choice.  Nothing here needs the host to know
// how many rows an expert got: the grouped GEMM is launched with an upper
// bound of row tiles and every workgroup finds its (expert, tile) from the
// offsets, so a step can be captured in a HIP graph.
//
// Router arithmetic (sigmoid, correction, group sums, comparisons) is fp32.
// GEMMs take bf16 (v_mfma_f32_16x16x16_bf16) or fp32 (v_mfma_f32_16x16x4_f32,
// true fp32 products) operands and accumulate in fp32.
#include "../kernels/common.h"

namespace {

// (value, index) argmax over a wave; ties go to the lower index
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, 64);
    const int oi = __shfl_xor(i, o, 64);
    if (ov > v || (ov == v && oi < i)) {
      v = ov;
      i = oi;
    }
  }
}

// One wave per token.  c[e] = s[e] + corr[e] are the choice scores, s = sigmoid(z)
// or softmax(z) over all experts; with n_groups > 1 only the experts of the `keep`
// groups with the largest group score (the sum of their two best choice scores,
// or with group_max their best) compete; the `top` best are written with weight
// s (no correction).
constexpr int kRouteWaves = 4;
__global__ void __launch_bounds__(64 * kRouteWaves) moe_route_kernel(int* __restrict__ idx, float* __restrict__ w,
                                                                     const float* __restrict__ z,
                                                                     const float* __restrict__ corr, int T, int E,
                                                                     int top, int n_groups, int keep, int score,
                                                                     int group_max) {
  extern __shared__ float sm[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * kRouteWaves + wv;
  const bool on = t < T;
  float* c = sm + wv * (E + n_groups);
  float* gs = c + E;
  const float* zt = z + (on ? t : 0) * E;
  // score 0: s = sigmoid(z); 1: s = softmax(z) over all experts (zmax, zinv: its maximum and 1 / sum)
  float zmax = 0.f, zinv = 1.f;
  if (score == 1) {
    float mxv = -INFINITY;
    for (int e = lane; e < E; e += 64) mxv = fmaxf(mxv, zt[e]);
    zmax = wave_reduce_max(mxv);
    float sm_ = 0.f;
    for (int e = lane; e < E; e += 64) sm_ += expf(zt[e] - zmax);
    zinv = 1.f / wave_reduce_sum(sm_);
  }
  for (int e = lane; e < E; e += 64)
    c[e] = (score == 1 ? expf(zt[e] - zmax) * zinv : 1.f / (1.f + expf(-zt[e]))) + (corr ? corr[e] : 0.f);
  __syncthreads();
  if (n_groups > 1) {
    const int per = E / n_groups;
    for (int g = lane; g < n_groups; g += 64) {
      float a = -INFINITY, b = -INFINITY;  // two largest
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float v = c[e];
        if (v > a) {
          b = a;
          a = v;
        } else if (v > b) {
          b = v;
        }
      }
      gs[g] = per > 1 && !group_max ? a + b : a;
    }
    __syncthreads();
    for (int k = 0; k < keep; ++k) {  // kept groups are marked +inf
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < n_groups; g += 64) {
        const float v = gs[g];
        if (v != INFINITY && (v > bv || (v == bv && g < bi))) {
          bv = v;
          bi = g;
        }
      }
      wave_argmax(bv, bi);
      __syncthreads();
      if (lane == 0 && bi < n_groups) gs[bi] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < E; e += 64)
      if (gs[e / per] != INFINITY) c[e] = -INFINITY;
    __syncthreads();
  }
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = c[e];
      if (v > bv || (v == bv && e < bi && v != -INFINITY)) {
        bv = v;
        bi = e;
      }
    }
    wave_argmax(bv, bi);
    if (bi >= E) bi = 0;  // nothing left to choose (rejected on the host)
    __syncthreads();
    if (lane == 0) {
      c[bi] = -INFINITY;
      if (on) {
        idx[t * top + k] = bi;
        w[t * top + k] = score == 1 ? expf(zt[bi] - zmax) * zinv : 1.f / (1.f + expf(-zt[bi]));
      }
    }
    __syncthreads();
  }
}

// order [R]: slots sorted by expert, stable; offsets [E + 1].  One workgroup:
// counts by LDS atomics (the counts do not depend on their order), a serial
// scan over the experts, then every wave places the slots of its experts in
// slot order with ballots.  STAGE: the choices are first copied into LDS as
// bytes (E <= 256, R <= kPlanStage), so the placement passes read no global
// memory.
constexpr int kPlanThreads = 1024;
constexpr int kPlanStage = 48 * 1024;
template <bool STAGE>
__global__ void __launch_bounds__(kPlanThreads) moe_plan_kernel(int* __restrict__ order, int* __restrict__ offsets,
                                                                const int* __restrict__ idx, int R, int E) {
  extern __shared__ int ism[];
  int* cnt = ism;
  int* base = ism + E;
  unsigned char* mine = reinterpret_cast<unsigned char*>(ism + 2 * E + 1);
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  for (int e = tid; e < E; e += kPlanThreads) cnt[e] = 0;
  __syncthreads();
  for (int r = tid; r < R; r += kPlanThreads) {
    const int e = idx[r];
    const bool ok = e >= 0 && e < E;
    if (ok) atomicAdd(&cnt[e], 1);
    if constexpr (STAGE) mine[r] = ok ? (unsigned char)e : 0;  // choices outside the experts are rejected by route
  }
  __syncthreads();
  if (tid == 0) {
    int acc = 0;
    for (int e = 0; e < E; ++e) {
      base[e] = acc;
      acc += cnt[e];
    }
    base[E] = acc;
  }
  __syncthreads();
  for (int e = tid; e <= E; e += kPlanThreads) offsets[e] = base[e];
  for (int e = wv; e < E; e += kPlanThreads / 64) {
    int at = base[e];
    for (int r0 = 0; r0 < R; r0 += 64) {
      const int r = r0 + lane;
      bool hit;
      if constexpr (STAGE) hit = r < R && mine[r] == e;
      else hit = r < R && idx[r] == e;
      const unsigned long long m = __builtin_amdgcn_ballot_w64(hit);
      if (hit) order[at + __builtin_popcountll(m & ((1ull << lane) - 1ull))] = r;
      at += __builtin_popcountll(m);
    }
  }
}

// ---------------------------------------------------------------------------
// Grouped GEMM.  For expert e, rows r in [offsets[e], offsets[e + 1]):
//     out[dst(r), :] = a[src(r), :] @ w[e]^T        w [E, N, K]
// src(r) = order[r] / top (gather: a has one row per token) or r; dst(r) =
// order[r] (scatter: slot order) or r.  A workgroup (4 waves) computes a
// 64-row x 64-column tile; K runs in steps of 32 through LDS, the next step's
// global loads in flight during the products.  The products are swapped,
// C^T = W A^T, so a lane ends up with four neighbouring columns of one row.
constexpr int kTM = 64, kTN = 64, kTK = 32;

template <typename T> struct Frag;
template <> struct Frag<bf16_t> {
  static constexpr int kPad = 8;
  __device__ static __forceinline__ f32x4 mma(const bf16_t* wp, const bf16_t* ap, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const i16x4*>(wp),
                                                     *reinterpret_cast<const i16x4*>(ap), c, 0, 0, 0);
  }
  __device__ static __forceinline__ void store4(bf16_t* o, f32x4 v, int n) {
    if (n >= 4 && (uintptr_t)o % 8 == 0) {
      uint2 p;
      p.x = pack_bf16x2(v[0], v[1]);
      p.y = pack_bf16x2(v[2], v[3]);
      *reinterpret_cast<uint2*>(o) = p;
    } else {
      for (int i = 0; i < n && i < 4; ++i) o[i] = f32_to_bf16(v[i]);
    }
  }
};
template <> struct Frag<float> {
  static constexpr int kPad = 4;
  // the four lane groups supply k = 4 g + s in step s: every k of the 16 once
  __device__ static __forceinline__ f32x4 mma(const float* wp, const float* ap, f32x4 c) {
#pragma unroll
    for (int s = 0; s < 4; ++s) c = __builtin_amdgcn_mfma_f32_16x16x4f32(wp[s], ap[s], c, 0, 0, 0);
    return c;
  }
  __device__ static __forceinline__ void store4(float* o, f32x4 v, int n) {
    if (n >= 4 && (uintptr_t)o % 16 == 0) {
      *reinterpret_cast<f32x4*>(o) = v;
    } else {
      for (int i = 0; i < n && i < 4; ++i) o[i] = v[i];
    }
  }
};

// eight consecutive elements of a row, zeros past `left` (elements left in the row)
template <typename T> struct Oct {
  T v[8];
  __device__ __forceinline__ void load(const T* p, int left, bool on) {
    if (on && left >= 8 && (uintptr_t)p % 16 == 0) {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      u32x4* d = reinterpret_cast<u32x4*>(v);
      const u32x4* s = reinterpret_cast<const u32x4*>(p);
      d[0] = s[0];
      if constexpr (sizeof(T) == 4) d[1] = s[1];
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = (on && i < left) ? p[i] : (T)0;
    }
  }
  __device__ __forceinline__ void store(T* p) const {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4* s = reinterpret_cast<const u32x4*>(v);
    u32x4* d = reinterpret_cast<u32x4*>(p);
    d[0] = s[0];
    if constexpr (sizeof(T) == 4) d[1] = s[1];
  }
};

template <typename T>
__global__ void __launch_bounds__(256) grouped_gemm_kernel(T* __restrict__ out, const T* __restrict__ a,
                                                           int64_t a_stride, const T* __restrict__ w,
                                                           const int* __restrict__ order,
                                                           const int* __restrict__ offsets, int E, int N, int K,
                                                           int top, int gather, int scatter) {
  constexpr int kStride = kTK + Frag<T>::kPad;
  __shared__ __attribute__((aligned(16))) T As[kTM * kStride];
  __shared__ __attribute__((aligned(16))) T Ws[kTN * kStride];
  // this workgroup's expert and row tile
  int tile = blockIdx.x, e = 0, lo = 0, hi = 0;
  for (; e < E; ++e) {
    lo = offsets[e];
    hi = offsets[e + 1];
    const int nt = (hi - lo + kTM - 1) / kTM;
    if (tile < nt) break;
    tile -= nt;
  }
  if (e >= E) return;
  const int row0 = lo + tile * kTM;
  const int rows = hi - row0 < kTM ? hi - row0 : kTM;
  const int n0 = blockIdx.y * kTN;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int c16 = lane & 15, g4 = lane >> 4;
  // staging: thread t moves eight k-elements (t % 4) of row t / 4 of both tiles
  const int sr = tid >> 2, sk = (tid & 3) * 8;
  const bool a_on = sr < rows;
  const int ar = row0 + (a_on ? sr : 0);
  const int64_t src = gather ? order[ar] / top : ar;
  const T* ap = a + src * a_stride + sk;
  const bool w_on = n0 + sr < N;
  const T* wp = w + ((int64_t)e * N + (w_on ? n0 + sr : 0)) * K + sk;
  const int wm = wv >> 1, wn = wv & 1;  // this wave: rows 32 wm .., columns 32 wn ..
  f32x4 C[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) C[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  Oct<T> ra, rw;
  ra.load(ap, K - sk, a_on);
  rw.load(wp, K - sk, w_on);
  for (int k0 = 0; k0 < K; k0 += kTK) {
    ra.store(As + sr * kStride + sk);
    rw.store(Ws + sr * kStride + sk);
    __syncthreads();
    if (k0 + kTK < K) {
      ra.load(ap + k0 + kTK, K - (k0 + kTK + sk), a_on);
      rw.load(wp + k0 + kTK, K - (k0 + kTK + sk), w_on);
    }
#pragma unroll
    for (int kk = 0; kk < kTK; kk += 16) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const T* wf = Ws + (32 * wn + 16 * j + c16) * kStride + kk + 4 * g4;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const T* af = As + (32 * wm + 16 * i + c16) * kStride + kk + 4 * g4;
          C[i][j] = Frag<T>::mma(wf, af, C[i][j]);
        }
      }
    }
    __syncthreads();
  }
  // C[i][j]: row 32 wm + 16 i + c16, columns n0 + 32 wn + 16 j + 4 g4 .. + 3
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = 32 * wm + 16 * i + c16;
    if (m >= rows) continue;
    const int64_t dst = scatter ? order[row0 + m] : row0 + m;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + 32 * wn + 16 * j + 4 * g4;
      if (n < N) Frag<T>::store4(out + dst * N + n, C[i][j], N - n);
    }
  }
}

// out[t, :] = sum_k wgt[t, k] * y[t * top + k, :] (+ shared[t, :]), fp32 sum in the order of k;
// V elements (16 bytes) per thread and access, V = 1 for unaligned widths
template <typename T, int V>
__global__ void __launch_bounds__(256) moe_combine_kernel(T* __restrict__ out, const T* __restrict__ y,
                                                          const float* __restrict__ wgt, const T* __restrict__ shared,
                                                          int64_t sh_stride, int top, int W) {
  const int64_t t = blockIdx.x;
  auto load = [](const T* p, float* f) {
    if constexpr (V == 1) {
      if constexpr (sizeof(T) == 2) f[0] = bf16_to_f32(p[0]); else f[0] = p[0];
    } else if constexpr (sizeof(T) == 2) {
      const u16x8 a = *reinterpret_cast<const u16x8*>(p);
#pragma unroll
      for (int i = 0; i < 4; ++i) f[2 * i] = bf16lo(a.w[i]), f[2 * i + 1] = bf16hi(a.w[i]);
    } else {
      const f32x4 a = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
      for (int i = 0; i < 4; ++i) f[i] = a[i];
    }
  };
  for (int c = threadIdx.x * V; c < W; c += 256 * V) {
    float acc[V], f[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = 0.f;
    for (int k = 0; k < top; ++k) {
      load(y + (t * top + k) * (int64_t)W + c, f);
      const float g = wgt[t * top + k];
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] += g * f[i];
    }
    if (shared) {
      load(shared + t * sh_stride + c, f);
#pragma unroll
      for (int i = 0; i < V; ++i) acc[i] += f[i];
    }
    T* o = out + t * (int64_t)W + c;
    if constexpr (V == 1) {
      if constexpr (sizeof(T) == 2) o[0] = f32_to_bf16(acc[0]); else o[0] = acc[0];
    } else if constexpr (sizeof(T) == 2) {
      u16x8 r;
#pragma unroll
      for (int i = 0; i < 4; ++i) r.w[i] = pack_bf16x2(acc[2 * i], acc[2 * i + 1]);
      *reinterpret_cast<u16x8*>(o) = r;
    } else {
      *reinterpret_cast<f32x4*>(o) = f32x4{acc[0], acc[1], acc[2], acc[3]};
    }
  }
}

}  // namespace

extern "C" {

int dxm_moe_route(int* idx, float* w, const float* z, const float* corr, int T, int E, int top, int n_groups,
                  int keep, int score, int group_max, hipStream_t st) {
  if (T <= 0) return 0;
  if (score < 0 || score > 1) return 3;
  if (E < 1 || n_groups < 1 || E % n_groups || keep < 1 || keep > n_groups || top < 1 ||
      top > keep * (E / n_groups))
    return 1;
  const size_t lds = (size_t)kRouteWaves * (E + n_groups) * sizeof(float);
  if (lds > 48 * 1024) return 2;
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + kRouteWaves - 1) / kRouteWaves), dim3(64 * kRouteWaves), lds, st, idx,
                     w, z, corr, T, E, top, n_groups, keep, score, group_max);
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_moe_plan(int* order, int* offsets, const int* idx, int R, int E, hipStream_t st) {
  if (E < 1 || R < 0) return 1;
  const size_t lds = (size_t)(2 * E + 1) * sizeof(int);
  if (lds > 12 * 1024) return 2;
  if (E <= 256 && R <= kPlanStage)
    hipLaunchKernelGGL(moe_plan_kernel<true>, dim3(1), dim3(kPlanThreads), lds + R, st, order, offsets, idx, R, E);
  else
    hipLaunchKernelGGL(moe_plan_kernel<false>, dim3(1), dim3(kPlanThreads), lds, st, order, offsets, idx, R, E);
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_grouped_gemm(void* out, const void* a, int64_t a_stride, const void* w, const int* order, const int* offsets,
                     int R, int E, int N, int K, int top, int gather, int scatter, int f32, hipStream_t st) {
  if (R <= 0) return 0;
  if (E < 1 || N < 1 || K < 1 || top < 1) return 1;
  const unsigned tiles = (unsigned)((R + kTM - 1) / kTM + E);  // at most this many row tiles over all experts
  const unsigned ny = (unsigned)((N + kTN - 1) / kTN);
  if (ny > 65535) return 2;
  if (f32)
    hipLaunchKernelGGL(grouped_gemm_kernel<float>, dim3(tiles, ny), dim3(256), 0, st, (float*)out, (const float*)a,
                       a_stride, (const float*)w, order, offsets, E, N, K, top, gather, scatter);
  else
    hipLaunchKernelGGL(grouped_gemm_kernel<bf16_t>, dim3(tiles, ny), dim3(256), 0, st, (bf16_t*)out, (const bf16_t*)a,
                       a_stride, (const bf16_t*)w, order, offsets, E, N, K, top, gather, scatter);
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_moe_combine(void* out, const void* y, const float* wgt, const void* shared, int64_t sh_stride, int T, int top,
                    int W, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (top < 1 || W < 1) return 1;
  const int per = f32 ? 4 : 8;  // elements per 16 bytes
  const bool vec = W % per == 0 && sh_stride % per == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)y % 16 == 0 &&
                   (uintptr_t)shared % 16 == 0;
  if (f32) {
    if (vec)
      hipLaunchKernelGGL((moe_combine_kernel<float, 4>), dim3(T), dim3(256), 0, st, (float*)out, (const float*)y, wgt,
                         (const float*)shared, sh_stride, top, W);
    else
      hipLaunchKernelGGL((moe_combine_kernel<float, 1>), dim3(T), dim3(256), 0, st, (float*)out, (const float*)y, wgt,
                         (const float*)shared, sh_stride, top, W);
  } else {
    if (vec)
      hipLaunchKernelGGL((moe_combine_kernel<bf16_t, 8>), dim3(T), dim3(256), 0, st, (bf16_t*)out, (const bf16_t*)y,
                         wgt, (const bf16_t*)shared, sh_stride, top, W);
    else
      hipLaunchKernelGGL((moe_combine_kernel<bf16_t, 1>), dim3(T), dim3(256), 0, st, (bf16_t*)out, (const bf16_t*)y,
                         wgt, (const bf16_t*)shared, sh_stride, top, W);
  }
  DX_CHECK_LAUNCH();
  return 0;
}

}  // extern "C"
