// Paged softmax attention, one wave per (token row, query head), for gfx950.
//
// The general kernel of the layer-listed models: every size is a run-time
// argument (query/key width d, value width dv, head counts, maps), rows of one
// launch may be prompt-chunk tokens and single decode tokens of different
// sequences side by side, and the visible keys of a row at position p are
//     causal:  0 .. p          window: max(0, p - size + 1) .. p
//     chunk:   floor(p / size) * size .. p
// and, for a window with `keep` > 0, also the sequence's first `keep` keys
// (0 .. keep - 1, at their true positions) however far back they lie,
// counted in sequence positions, so the result does not depend on how a prompt
// was cut into steps.  The score of query position p and key position j is
// s = q . k * scale, optionally capped, s <- cap * tanh(s / cap), and optionally
// lowered by a per-head penalty that grows with the logarithm of the distance,
// s <- s - r1[qh] * ln(1 + r2[qh] * (p - j)).  Scores, softmax weights and the weighted sum are fp32;
// q, the caches and the output are bf16 or fp32 (the output optionally fp32
// beside bf16 caches).
//
// Caches are token-major: K [slots, Wk], V [slots, Wv], slot = block * bs +
// offset.  Query head qh of `maps` maps per head reads K head
// (qh / maps / group) * maps + qh % maps and V head qh / maps / group
// (group = query heads per key/value head): maps = 1 is grouped-query
// attention, maps = 2 the two score maps of differential attention.
//
// With `sink` (a number per query vector) a softmax's denominator also holds
// exp(sink): a key without a value that is neither scaled nor masked, counted once.
//
// Work split: 64 keys per tile, one key per lane for the scores (the query
// sits in LDS as fp32, pre-scaled), then the lanes turn to the value columns
// (lane + 64 c) for the weighted sum, the weights broadcast by readlane.
// `parts` > 1 splits a row's keys over blockIdx.z (long decode contexts); the
// partial (max, sum, acc) go to a workspace and merge_parts_kernel joins them.
#include "../kernels/common.h"

namespace {

template <typename T> struct Elem;
template <> struct Elem<bf16_t> {
  static constexpr int kVec = 8;
  __device__ static __forceinline__ float ld(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
  __device__ static __forceinline__ void st(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
  __device__ static __forceinline__ float dot(const bf16_t* k, const float* q) {
    const u16x8 a = *reinterpret_cast<const u16x8*>(k);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) s += bf16lo(a.w[i]) * q[2 * i] + bf16hi(a.w[i]) * q[2 * i + 1];
    return s;
  }
};
template <> struct Elem<float> {
  static constexpr int kVec = 4;
  __device__ static __forceinline__ float ld(const float* p, int64_t i) { return p[i]; }
  __device__ static __forceinline__ void st(float* p, int64_t i, float v) { p[i] = v; }
  __device__ static __forceinline__ float dot(const float* k, const float* q) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(k);
    return a[0] * q[0] + a[1] * q[1] + a[2] * q[2] + a[3] * q[3];
  }
};

struct RowAttnArgs {
  const void* q;
  int64_t q_stride;  // elements between token rows
  const void* kc;
  const void* vc;
  void* out;  // [rows, Hq, dv]
  float* ws;  // parts > 1: [rows, Hq, parts, 2 + dv]
  const int64_t* pos;
  const int* seq;  // row -> block-table row; null: row i is sequence i
  const int* bt;
  int bt_stride;
  int bs;
  int n_qh, maps, group;
  int d, dv, Wk, Wv;
  float scale;
  int mask;  // 0 causal, 1 window, 2 chunk
  int size;
  int parts;
  float softcap;    // 0: scores are not capped
  const float* r1;  // [n_qh] distance penalty (null: none)
  const float* r2;
  int wfn;              // 0: softmax over the visible keys; 1: sigmoid(s) per visible key, not normalised
  const float* hbias;   // [n_qh] added to the score (null: none)
  const void* gate;     // [rows, gate_stride] logits per head: the result is multiplied by sigmoid (null: none)
  int64_t gate_stride;
  int keep;           // window mask: the first `keep` keys of the sequence stay visible (0: none)
  const float* sink;  // [n_qh] softmax only: exp(sink) joins the denominator (null: none)
};

template <typename T, typename OutT, int NV>
__global__ void __launch_bounds__(64) row_attention_kernel(RowAttnArgs a) {
  extern __shared__ float qs[];  // [d]
  const int lane = threadIdx.x;
  const int qh = blockIdx.x, row = blockIdx.y, part = blockIdx.z;
  const int64_t p = a.pos[row];
  const int sq = a.seq ? a.seq[row] : row;
  const int* bt = a.bt + (int64_t)sq * a.bt_stride;
  const int head = qh / a.maps, m = qh - head * a.maps, g = head / a.group;
  const int kh = g * a.maps + m;
  int64_t lo = 0;
  if (a.mask == 1) lo = p - a.size + 1 > 0 ? p - a.size + 1 : 0;
  if (a.mask == 2) lo = p / a.size * a.size;
  const T* q = (const T*)a.q + (int64_t)row * a.q_stride + (int64_t)qh * a.d;
  for (int e = lane; e < a.d; e += 64) qs[e] = Elem<T>::ld(q, e) * a.scale;
  __syncthreads();
  const T* kc = (const T*)a.kc + (int64_t)kh * a.d;
  const T* vc = (const T*)a.vc + (int64_t)g * a.dv;
  // visible keys in one numbering u = 0 .. n_keys - 1: the kept first nf keys, then lo .. p
  const int64_t nf = a.mask == 1 && a.keep > 0 ? (a.keep < lo ? a.keep : lo) : 0;
  const int64_t n_keys = nf + p - lo + 1;
  const int64_t tiles = (n_keys + 63) / 64;
  const int64_t tpp = (tiles + a.parts - 1) / a.parts;
  const int64_t t0 = part * tpp, t1 = t0 + tpp < tiles ? t0 + tpp : tiles;
  const bool vec = a.d % Elem<T>::kVec == 0 && a.Wk % Elem<T>::kVec == 0;
  const float cap = a.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  const float r1 = a.r1 ? a.r1[qh] : 0.f, r2 = a.r1 ? a.r2[qh] : 0.f;
  const float hb = a.hbias ? a.hbias[qh] : 0.f;
  float mx = a.wfn ? 0.f : -INFINITY, l = a.wfn ? 1.f : 0.f;
  float acc[NV];
#pragma unroll
  for (int c = 0; c < NV; ++c) acc[c] = 0.f;
  for (int64_t t = t0; t < t1; ++t) {
    const int64_t u = t * 64 + lane;
    const int64_t j = u < nf ? u : lo + (u - nf);
    const bool ok = u < n_keys;
    int slot = 0;
    float s = -INFINITY;
    if (ok) {
      slot = bt[j / a.bs] * a.bs + (int)(j % a.bs);
      const T* k = kc + (int64_t)slot * a.Wk;
      float sum = 0.f;
      if (vec) {
        for (int e = 0; e < a.d; e += Elem<T>::kVec) sum += Elem<T>::dot(k + e, qs + e);
      } else {
        for (int e = 0; e < a.d; ++e) sum += Elem<T>::ld(k, e) * qs[e];
      }
      if (cap > 0.f) sum = cap * tanhf(sum * inv_cap);
      if (a.r1) sum -= r1 * log1pf(r2 * (float)(p - j));
      s = sum + hb;
    }
    float w;
    if (a.wfn) {  // every visible key weighs sigmoid(s); nothing to rescale
      w = ok ? 1.f / (1.f + expf(-s)) : 0.f;
    } else {
      const float mn = fmaxf(mx, wave_reduce_max(s));
      w = ok ? __expf(s - mn) : 0.f;
      const float alpha = __expf(mx - mn);  // first tile: exp(-inf) = 0
      l = l * alpha + wave_reduce_sum(w);
      mx = mn;
#pragma unroll
      for (int c = 0; c < NV; ++c) acc[c] *= alpha;
    }
    const int64_t left = n_keys - t * 64;
    const int n = left < 64 ? (int)left : 64;
    for (int jj = 0; jj < n; ++jj) {
      const float wj = __shfl(w, jj, 64);
      const int sj = __shfl(slot, jj, 64);
      const T* v = vc + (int64_t)sj * a.Wv;
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        const int e = lane + 64 * c;
        if (e < a.dv) acc[c] += wj * Elem<T>::ld(v, e);
      }
    }
  }
  if (a.parts == 1) {
    OutT* o = (OutT*)a.out + ((int64_t)row * a.n_qh + qh) * a.dv;
    if (a.sink && !a.wfn) l += expf(a.sink[qh] - mx);
    float inv = 1.f / l;
    if (a.gate) inv /= 1.f + expf(-Elem<T>::ld((const T*)a.gate, (int64_t)row * a.gate_stride + head));
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int e = lane + 64 * c;
      if (e < a.dv) Elem<OutT>::st(o, e, acc[c] * inv);
    }
  } else {
    float* w = a.ws + (((int64_t)row * a.n_qh + qh) * a.parts + part) * (2 + a.dv);
    if (lane == 0) {
      w[0] = mx;
      w[1] = l;
    }
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int e = lane + 64 * c;
      if (e < a.dv) w[2 + e] = acc[c];
    }
  }
}

// joins the per-part (max, sum, acc) of one (row, head): one wave each
// (sigmoid weights: every part carries max 0 and sum 1, so the join is the plain sum of the
// parts divided by their number -- `plain` undoes that division); gate: logits [rows, gs] per
// head, the result is multiplied by their sigmoid; sink: [n_qh], exp(sink) joins the softmax denominator once
template <typename OutT, typename GT>
__global__ void __launch_bounds__(64) merge_parts_kernel(OutT* __restrict__ out, const float* __restrict__ ws,
                                                         int parts, int dv, int plain, const GT* __restrict__ gate,
                                                         int64_t gs, int n_qh, int maps,
                                                         const float* __restrict__ sink) {
  const int lane = threadIdx.x;
  const int64_t v = blockIdx.x;
  const float* w = ws + v * parts * (int64_t)(2 + dv);
  float post = plain ? (float)parts : 1.f;
  if (gate) {
    const int64_t row = v / n_qh;
    const int head = (int)(v - row * n_qh) / maps;
    post /= 1.f + expf(-Elem<GT>::ld(gate, row * gs + head));
  }
  float mx = -INFINITY;
  for (int p = 0; p < parts; ++p) mx = fmaxf(mx, w[(int64_t)p * (2 + dv)]);
  float l = 0.f;
  for (int p = 0; p < parts; ++p) {
    const float* wp = w + (int64_t)p * (2 + dv);
    if (wp[1] > 0.f) l += wp[1] * __expf(wp[0] - mx);
  }
  if (sink && !plain) l += expf(sink[v % n_qh] - mx);
  const float inv = post / l;
  for (int e = lane; e < dv; e += 64) {
    float acc = 0.f;
    for (int p = 0; p < parts; ++p) {
      const float* wp = w + (int64_t)p * (2 + dv);
      if (wp[1] > 0.f) acc += wp[2 + e] * __expf(wp[0] - mx);
    }
    Elem<OutT>::st(out, v * dv + e, acc * inv);
  }
}

template <typename T, typename OutT>
int launch_rows(const RowAttnArgs& a, int rows, hipStream_t st) {
  const int nv = (a.dv + 63) / 64;
  const size_t lds = (size_t)a.d * sizeof(float);
  for (int r0 = 0; r0 < rows; r0 += 65535) {
    RowAttnArgs b = a;
    const int nr = rows - r0 < 65535 ? rows - r0 : 65535;
    b.q = (const T*)a.q + (int64_t)r0 * a.q_stride;
    b.out = (OutT*)a.out + (int64_t)r0 * a.n_qh * a.dv;
    b.ws = a.ws ? a.ws + (int64_t)r0 * a.n_qh * a.parts * (2 + a.dv) : nullptr;
    b.pos = a.pos + r0;
    b.seq = a.seq ? a.seq + r0 : nullptr;
    if (!a.seq && r0) return 5;  // implicit row == sequence numbering cannot be offset
    b.gate = a.gate ? (const T*)a.gate + (int64_t)r0 * a.gate_stride : nullptr;
    const dim3 grid(a.n_qh, nr, a.parts);
    if (nv <= 1) hipLaunchKernelGGL((row_attention_kernel<T, OutT, 1>), grid, dim3(64), lds, st, b);
    else if (nv <= 2) hipLaunchKernelGGL((row_attention_kernel<T, OutT, 2>), grid, dim3(64), lds, st, b);
    else if (nv <= 4) hipLaunchKernelGGL((row_attention_kernel<T, OutT, 4>), grid, dim3(64), lds, st, b);
    else if (nv <= 8) hipLaunchKernelGGL((row_attention_kernel<T, OutT, 8>), grid, dim3(64), lds, st, b);
    else hipLaunchKernelGGL((row_attention_kernel<T, OutT, 16>), grid, dim3(64), lds, st, b);
    if (a.parts > 1)
      hipLaunchKernelGGL((merge_parts_kernel<OutT, T>), dim3((unsigned)nr * a.n_qh), dim3(64), 0, st, (OutT*)b.out, b.ws,
                         a.parts, a.dv, a.wfn, (const T*)b.gate, a.gate_stride, a.n_qh, a.maps, a.sink);
  }
  DX_CHECK_LAUNCH();
  return 0;
}

}  // namespace

extern "C" int dxm_row_attention(void* out, float* ws, const void* q, int64_t q_stride, const void* kc, const void* vc,
                                 const int64_t* pos, const int* seq, const int* bt, int bt_stride, int bs, int rows,
                                 int n_qh, int maps, int group, int d, int dv, int Wk, int Wv, float scale, int mask,
                                 int size, float softcap, const float* r1, const float* r2, int wfn, const float* hbias,
                                 const void* gate, int64_t gate_stride, int keep, const float* sink, int parts, int f32,
                                 int out_f32, hipStream_t st) {
  if (rows <= 0) return 0;
  if (n_qh < 1 || maps < 1 || group < 1 || n_qh % maps || (n_qh / maps) % group) return 1;
  if (d < 1 || dv < 1 || dv > 1024 || d > 8192) return 2;
  if (mask < 0 || mask > 2 || (mask && size < 1) || parts < 1 || parts > 65535 || n_qh > 65535) return 3;
  if (parts > 1 && !ws) return 4;
  if (softcap < 0.f || (r1 && !r2) || wfn < 0 || wfn > 1 || keep < 0 || (keep && mask != 1)) return 6;
  RowAttnArgs a{q, q_stride, kc, vc, out, ws, pos, seq, bt, bt_stride, bs, n_qh, maps, group,
                d, dv, Wk, Wv, scale, mask, size, parts, softcap, r1, r2, wfn, hbias, gate, gate_stride, keep, sink};
  if (f32) return launch_rows<float, float>(a, rows, st);
  if (out_f32) return launch_rows<bf16_t, float>(a, rows, st);
  return launch_rows<bf16_t, bf16_t>(a, rows, st);
}

// out [n_vec, dv] (bf16 or fp32) from per-part partials ws [n_vec, parts, 2 + dv]; n_vec = rows * n_qh;
// plain: the parts hold sigmoid-weighted sums (max 0, sum 1 each); gate: bf16 logits [rows, gate_stride]
extern "C" int dxm_merge_parts(void* out, const float* ws, int64_t n_vec, int parts, int dv, int plain,
                               const void* gate, int64_t gate_stride, int n_qh, int maps, const float* sink,
                               int out_f32, hipStream_t st) {
  if (n_vec <= 0) return 0;
  if (parts < 1 || dv < 1 || n_vec > 0x7fffffff || n_qh < 1 || maps < 1) return 1;
  if (out_f32)
    hipLaunchKernelGGL((merge_parts_kernel<float, bf16_t>), dim3((unsigned)n_vec), dim3(64), 0, st, (float*)out, ws,
                       parts, dv, plain, (const bf16_t*)gate, gate_stride, n_qh, maps, sink);
  else
    hipLaunchKernelGGL((merge_parts_kernel<bf16_t, bf16_t>), dim3((unsigned)n_vec), dim3(64), 0, st, (bf16_t*)out, ws,
                       parts, dv, plain, (const bf16_t*)gate, gate_stride, n_qh, maps, sink);
  DX_CHECK_LAUNCH();
  return 0;
}
