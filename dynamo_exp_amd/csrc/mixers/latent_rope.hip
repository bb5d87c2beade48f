// Query / key preparation of latent attention with a rotated key part, for
// gfx950: per token row
//   * the latent (the first r columns of the down-projection) is RMS-normed with
//     a weight per column and written to the paged cache row [0, r);
//   * the key part that carries the position (the next dr columns, not normed,
//     shared by all heads) is rotated and written to the cache row [r, r + dr);
//   * every head's query is assembled as [qa_h (r) | rotate(q_h's last dr columns)]:
//     qa is the head's unrotated query part already multiplied by the head's key
//     up-projection, so that q' . [latent | rotated key] is the head's score.
// The cache row [latent | rotated key] is key and (its first r columns) value
// of one shared head.
//
// Rotation: the first 2 * half columns of a dr-wide part, column i paired with
// i + half, angle = position * inv_freq[i] (fp32, sincosf), cosine and sine
// both multiplied by `mag`; columns from 2 * half on pass unchanged.
// Norm sums, angles and the rotation are fp32 whatever the element type is.
#include "../kernels/common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
template <> __device__ __forceinline__ float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <typename T> __device__ __forceinline__ void stf(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, int64_t i, float v) { p[i] = v; }

// VEC consecutive elements as floats, one 16-byte access
template <typename T, int V> struct VecIO;
template <> struct VecIO<bf16_t, 8> {
  __device__ static __forceinline__ void ld(const bf16_t* p, float* o) {
    const u16x8 a = *reinterpret_cast<const u16x8*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) o[2 * i] = bf16lo(a.w[i]), o[2 * i + 1] = bf16hi(a.w[i]);
  }
  __device__ static __forceinline__ void st(bf16_t* p, const float* v) {
    u16x8 a;
#pragma unroll
    for (int i = 0; i < 4; ++i) a.w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
    *reinterpret_cast<u16x8*>(p) = a;
  }
};
template <> struct VecIO<float, 4> {
  __device__ static __forceinline__ void ld(const float* p, float* o) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p);
    o[0] = a[0], o[1] = a[1], o[2] = a[2], o[3] = a[3];
  }
  __device__ static __forceinline__ void st(float* p, const float* v) {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
  }
};
template <typename T> struct VecIO<T, 1> {
  __device__ static __forceinline__ void ld(const T* p, float* o) { o[0] = ldf<T>(p, 0); }
  __device__ static __forceinline__ void st(T* p, const float* v) { stf<T>(p, 0, v[0]); }
};

struct LatentArgs {
  void* q_out;      // [T, H, r + dr]
  const void* qa;   // [H, T, r]: unrotated query parts times the key up-projection
  const void* q;    // [T, q_stride]: head h's rotated part at columns h * q_head + q_off .. + dr
  int64_t q_stride;
  int q_head, q_off;
  const void* kv;   // [T, kv_stride]: [latent (r) | rotated key part (dr)]
  int64_t kv_stride;
  const float* cn;  // [r] latent norm weight
  float eps;
  const float* inv_freq;  // [half]
  int half;
  float mag;
  const int64_t* pos;
  const int64_t* slots;  // cache row of every token (-1: not cached)
  void* cache;           // [slots, r + dr]
  int T, H, r, dr;
};

// VEC: elements per 16-byte chunk when r, dr, the rotated half, the row strides and the bases allow
// whole chunks (the query rows, the bulk of the bytes, are then built chunk by chunk), else 1
template <typename T, int VEC>
__global__ void __launch_bounds__(256) latent_rope_kernel(LatentArgs g) {
  extern __shared__ float cs_sn[];  // [half] cosines, [half] sines, both times mag
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const float p = (float)g.pos[t];
  for (int i = tid; i < g.half; i += blockDim.x) {
    float sn, cs;
    sincosf(p * g.inv_freq[i], &sn, &cs);
    cs_sn[i] = cs * g.mag;
    cs_sn[g.half + i] = sn * g.mag;
  }
  const T* kv = (const T*)g.kv + t * g.kv_stride;
  float ss = 0.f;
  for (int c = tid; c < g.r; c += blockDim.x) {
    const float x = ldf<T>(kv, c);
    ss += x * x;
  }
  const float rs = rsqrtf(block_reduce_sum(ss, red) / (float)g.r + g.eps);  // (also orders the LDS writes above)
  const int Wc = g.r + g.dr;
  // rotated value of column e (< dr) of a dr-wide part at src
  auto rot = [&](const T* src, int e) -> float {
    const float x = ldf<T>(src, e);
    if (e >= 2 * g.half) return x;
    const int i = e < g.half ? e : e - g.half;
    const float other = ldf<T>(src, e < g.half ? e + g.half : e - g.half);
    return e < g.half ? x * cs_sn[i] - other * cs_sn[g.half + i] : x * cs_sn[i] + other * cs_sn[g.half + i];
  };
  const int64_t slot = g.slots[t];
  if (slot >= 0) {
    T* row = (T*)g.cache + slot * Wc;
    for (int c = tid; c < g.r; c += blockDim.x) stf<T>(row, c, ldf<T>(kv, c) * rs * g.cn[c]);
    for (int e = tid; e < g.dr; e += blockDim.x) stf<T>(row, g.r + e, rot(kv + g.r, e));
  }
  const T* q = (const T*)g.q + t * g.q_stride;
  T* qo = (T*)g.q_out + t * (int64_t)g.H * Wc;
  if constexpr (VEC > 1) {
    // work items of VEC columns per head: copies of qa, rotated pairs of runs (a run of the low half
    // with its partner of the high half, every angle used once), runs that are not rotated
    typedef uint32_t raw4 __attribute__((ext_vector_type(4)));
    const int n_copy = g.r / VEC, n_pair = g.half / VEC, per = n_copy + n_pair + (g.dr - 2 * g.half) / VEC;
    for (int it = tid; it < g.H * per; it += blockDim.x) {
      const int h = it / per, j = it - h * per;
      T* dst = qo + (int64_t)h * Wc;
      const T* src = q + (int64_t)h * g.q_head + g.q_off;
      if (j < n_copy) {
        *reinterpret_cast<raw4*>(dst + j * VEC) =
            *reinterpret_cast<const raw4*>((const T*)g.qa + ((int64_t)h * g.T + t) * g.r + j * VEC);
      } else if (j < n_copy + n_pair) {
        const int e0 = (j - n_copy) * VEC;
        float x[VEC], y[VEC], lo[VEC], hi[VEC];
        VecIO<T, VEC>::ld(src + e0, x);
        VecIO<T, VEC>::ld(src + g.half + e0, y);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float cs = cs_sn[e0 + e], sn = cs_sn[g.half + e0 + e];
          lo[e] = x[e] * cs - y[e] * sn;
          hi[e] = y[e] * cs + x[e] * sn;
        }
        VecIO<T, VEC>::st(dst + g.r + e0, lo);
        VecIO<T, VEC>::st(dst + g.r + g.half + e0, hi);
      } else {
        const int e0 = 2 * g.half + (j - n_copy - n_pair) * VEC;
        *reinterpret_cast<raw4*>(dst + g.r + e0) = *reinterpret_cast<const raw4*>(src + e0);
      }
    }
  } else {
    for (int it = tid; it < g.H * Wc; it += blockDim.x) {
      const int h = it / Wc, c = it - h * Wc;
      if (c < g.r) qo[it] = ((const T*)g.qa)[((int64_t)h * g.T + t) * g.r + c];
      else stf<T>(qo, it, rot(q + (int64_t)h * g.q_head + g.q_off, c - g.r));
    }
  }
}

}  // namespace

extern "C" int dxm_latent_rope(void* q_out, const void* qa, const void* q, int64_t q_stride, int q_head, int q_off,
                               const void* kv, int64_t kv_stride, const float* cn, float eps, const float* inv_freq,
                               int half, float mag, const int64_t* pos, const int64_t* slots, void* cache, int T_, int H,
                               int r, int dr, int f32, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (H < 1 || r < 1 || dr < 0 || half < 0 || 2 * half > dr || half > 4096) return 1;
  if (!q_out || !qa || !kv || !cn || !pos || !slots || !cache || (dr && !q) || (half && !inv_freq)) return 2;
  if (q_off < 0 || q_off + dr > q_head) return 3;
  LatentArgs g{q_out, qa, q, q_stride, q_head, q_off, kv, kv_stride, cn, eps, inv_freq, half, mag,
               pos, slots, cache, T_, H, r, dr};
  const size_t lds = (size_t)2 * half * sizeof(float);
  const int V = f32 ? 4 : 8;
  const bool vec = r % V == 0 && dr % V == 0 && half % V == 0 && q_stride % V == 0 && q_head % V == 0 && q_off % V == 0 &&
                   (uintptr_t)q_out % 16 == 0 && (uintptr_t)qa % 16 == 0 && (uintptr_t)q % 16 == 0;
  if (f32 && vec) hipLaunchKernelGGL((latent_rope_kernel<float, 4>), dim3(T_), dim3(256), lds, st, g);
  else if (f32) hipLaunchKernelGGL((latent_rope_kernel<float, 1>), dim3(T_), dim3(256), lds, st, g);
  else if (vec) hipLaunchKernelGGL((latent_rope_kernel<bf16_t, 8>), dim3(T_), dim3(256), lds, st, g);
  else hipLaunchKernelGGL((latent_rope_kernel<bf16_t, 1>), dim3(T_), dim3(256), lds, st, g);
  DX_CHECK_LAUNCH();
  return 0;
}
