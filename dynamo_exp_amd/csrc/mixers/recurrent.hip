// Kernels with per-sequence state for gfx950: the generalized delta rule (a
// running matrix per head), retention (a fixed decay per head), short causal convolutions over time fused with
// rotary positions and the paged cache write, the convolution tail update, and
// the per-head unit-RMS + gate that follows a recurrent mixer.
//
// State lives in slots ([slots, ...] tensors); a step names the slot of each of
// its sequences (state_slots [n_seq], -1: a padding row that touches nothing)
// and the first row of each (seq_rows [n_seq + 1]; null: row i is sequence i).
// Rows of a sequence are consecutive positions.  A sequence whose first row of
// the step is at position 0 starts from zero state, whatever its slot held.
//
// Every kernel is a template over the activation element (bf16 bits or float);
// decays, removal rates, unit keys, the running matrix, angles and all sums are
// fp32 whatever the element is.  Sizes are run-time arguments.
#include "../kernels/common.h"

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p, int64_t i);
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p, int64_t i) { return bf16_to_f32(p[i]); }
template <> __device__ __forceinline__ float ldf<float>(const float* p, int64_t i) { return p[i]; }
template <typename T> __device__ __forceinline__ void stf(T* p, int64_t i, float v);
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, int64_t i, float v) { p[i] = f32_to_bf16(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, int64_t i, float v) { p[i] = v; }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }

// ---------------------------------------------------------------------------
// Generalized delta rule.  Per (sequence, head) a matrix S [dk, dv]:
//     S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,   o_t = S_t^T r_t
// with w_t = exp(-decay_scale * sigmoid(wl_t + w_bias)), a_t = sigmoid(al_t + a_bias),
// u_t = k_t / sqrt(sum(k_t^2) + key_eps).  Columns of S are independent, so a
// thread owns a tile of kRows consecutive rows x CT consecutive columns in
// registers (every row vector it reads from LDS serves CT columns), R
// neighbouring lanes share the columns and join their partial dot products by
// DPP lane exchanges (no LDS traffic), and a workgroup of NT threads owns
// NT / R * CT columns of one (sequence, head).  CT is 4 where the launch has
// waves to fill the chip twice over, else 2 or 1 (a few long prompts): a
// token's dependent chain leaves a lone wave on a SIMD waiting most of the
// time, so the launch wants at least two waves on every SIMD.  The
// state tensor is stored column-major per head ([slots, H, dv, dk]) so that a
// wave's state traffic is contiguous runs.  What the recurrence needs per
// token and key channel beside r and k -- the unit key u, the decay w and
// a * u -- is computed for all rows at once by delta_prep_kernel (fp32, [T, H,
// 3, dk]): it is elementwise work and would otherwise sit in the sequential
// chain.  Tokens are staged through LDS kTok at a time, fetched into registers
// one block ahead (the latency hides behind the current block's recurrence).
constexpr int kRows = 16;  // state rows per thread
constexpr int kTok = 8;    // tokens per staged block

struct DeltaArgs {
  float* out;    // [T, H * dv]
  float* state;  // [slots, H, dv, dk]
  const void *r, *k, *v;
  int64_t rs, ks, vs;  // row strides (elements)
  const float* prep;   // [T, H, 3, dk]: unit key, decay, removal rate * unit key
  const int64_t* pos;
  const int* seq_rows;  // null: row i is sequence i
  const int* slots;
  int n_slots, T, H, dk, dv;
};

template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
// sum over the R lanes of an aligned lane group (R <= 16), the result in every lane of the group:
// neighbours within a quad, the other pair of the quad, the other quad of a half row (half-row
// mirror: the quads already hold one value each), the other half of a row of 16 (row mirror)
template <int R> __device__ __forceinline__ float group_sum(float v) {
  if constexpr (R >= 2) v += dpp_f<0xB1>(v);
  if constexpr (R >= 4) v += dpp_f<0x4E>(v);
  if constexpr (R >= 8) v += dpp_f<0x141>(v);
  if constexpr (R >= 16) v += dpp_f<0x140>(v);
  return v;
}

// one wave per (row, head): u = k / sqrt(sum k^2 + key_eps), w = exp(-decay_scale sigmoid(wl + w_bias)),
// a u with a = sigmoid(al + a_bias)
template <typename T>
__global__ void __launch_bounds__(64) delta_prep_kernel(float* __restrict__ prep, const T* __restrict__ k, int64_t ks,
                                                        const T* __restrict__ a, int64_t as, const T* __restrict__ w,
                                                        int64_t ws, const float* __restrict__ a_bias,
                                                        const float* __restrict__ w_bias, float decay_scale,
                                                        float key_eps, int H, int dk) {
  const int64_t v = blockIdx.x, row = v / H;
  const int h = (int)(v - row * H), lane = threadIdx.x;
  const T* kp = k + row * ks + (int64_t)h * dk;
  float ss = 0.f;
  for (int ch = lane; ch < dk; ch += 64) {
    const float x = ldf<T>(kp, ch);
    ss += x * x;
  }
  const float inv = rsqrtf(wave_reduce_sum(ss) + key_eps);
  float* o = prep + v * 3 * dk;
  for (int ch = lane; ch < dk; ch += 64) {
    const float u = ldf<T>(kp, ch) * inv;
    const float ab = a_bias ? a_bias[h * dk + ch] : 0.f, wb = w_bias ? w_bias[h * dk + ch] : 0.f;
    o[ch] = u;
    o[dk + ch] = expf(-decay_scale * sigmoidf_(ldf<T>(w, row * ws + (int64_t)h * dk + ch) + wb));
    o[2 * dk + ch] = sigmoidf_(ldf<T>(a, row * as + (int64_t)h * dk + ch) + ab) * u;
  }
}

template <typename T, int R, int NT, int CT>
__global__ void __launch_bounds__(NT) delta_rule_kernel(DeltaArgs g) {
  constexpr int kCols = CT;
  constexpr int kGroups = NT / R;            // column tiles per workgroup
  constexpr int kWgCols = kGroups * kCols;   // columns per workgroup
  constexpr int kDkp = kRows * R;            // padded key width
  constexpr int kE = (kTok * kDkp + NT - 1) / NT;  // staged elements per thread and array
  constexpr int kEv = (kTok * kWgCols + NT - 1) / NT;
  __shared__ __attribute__((aligned(16))) float sr[kTok][kDkp];
  __shared__ __attribute__((aligned(16))) float sk[kTok][kDkp];
  __shared__ __attribute__((aligned(16))) float su[kTok][kDkp];
  __shared__ __attribute__((aligned(16))) float sw[kTok][kDkp];
  __shared__ __attribute__((aligned(16))) float sa[kTok][kDkp];
  __shared__ __attribute__((aligned(16))) float sv[kTok][kWgCols];
  const int tid = threadIdx.x, part = tid % R, grp = tid / R;
  const int s = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * kWgCols + grp * kCols;
  const int r0 = g.seq_rows ? g.seq_rows[s] : s;
  const int r1 = g.seq_rows ? g.seq_rows[s + 1] : s + 1;
  const int slot = g.slots[s];
  const int n = r1 - r0;
  if (n <= 0 || r0 < 0 || r1 > g.T) return;
  if (slot < 0 || slot >= g.n_slots) {  // padding rows: a defined result, no state
    if (part == 0)
      for (int t = r0; t < r1; ++t)
        for (int c = 0; c < kCols; ++c)
          if (j0 + c < g.dv) g.out[(int64_t)t * g.H * g.dv + h * g.dv + j0 + c] = 0.f;
    return;
  }
  // The thread's 16 rows are four quads, quad m at row (m * R + part) * 4: for one m the R lanes of a
  // group read R consecutive 16-byte pieces of a row vector, so a wave's LDS read touches every bank once
  // (16 consecutive rows per lane would put lanes 0, 2, 4, .. on the same banks).
  float* sp = g.state + (((int64_t)slot * g.H + h) * g.dv) * g.dk;  // + column * dk + row
  const bool fresh = g.pos[r0] == 0;
  int rq[kRows / 4];
#pragma unroll
  for (int m = 0; m < kRows / 4; ++m) rq[m] = (m * R + part) * 4;
  float S[kCols][kRows];
#pragma unroll
  for (int c = 0; c < kCols; ++c) {
#pragma unroll
    for (int q = 0; q < kRows; ++q) S[c][q] = 0.f;
    if (fresh || j0 + c >= g.dv) continue;
    const float* spc = sp + (int64_t)(j0 + c) * g.dk;
#pragma unroll
    for (int m = 0; m < kRows / 4; ++m) {
      if (g.dk % 4 == 0 && rq[m] + 4 <= g.dk) {
        const f32x4 x = *reinterpret_cast<const f32x4*>(spc + rq[m]);
        S[c][4 * m] = x[0], S[c][4 * m + 1] = x[1], S[c][4 * m + 2] = x[2], S[c][4 * m + 3] = x[3];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (rq[m] + e < g.dk) S[c][4 * m + e] = spc[rq[m] + e];
      }
    }
  }
  const T* pr = (const T*)g.r + (int64_t)h * g.dk;
  const T* pk = (const T*)g.k + (int64_t)h * g.dk;
  const float* pp = g.prep + (int64_t)h * 3 * g.dk;
  const T* pv = (const T*)g.v + (int64_t)h * g.dv + blockIdx.z * kWgCols;
  float fr[kE], fk[kE], fu[kE], fa[kE], fw[kE], fv[kEv];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int e = 0; e < kE; ++e) {
      const int idx = tid + e * NT, tt = idx / kDkp, ch = idx % kDkp;
      const bool ok = idx < kTok * kDkp && t0 + tt < n && ch < g.dk;
      const int64_t row = r0 + t0 + tt;
      const float* pq = pp + row * g.H * 3 * g.dk + ch;
      fr[e] = ok ? ldf<T>(pr, row * g.rs + ch) : 0.f;
      fk[e] = ok ? ldf<T>(pk, row * g.ks + ch) : 0.f;
      fu[e] = ok ? pq[0] : 0.f;
      fw[e] = ok ? pq[g.dk] : 0.f;
      fa[e] = ok ? pq[2 * g.dk] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < kEv; ++e) {
      const int idx = tid + e * NT, tt = idx / kWgCols, cc = idx % kWgCols;
      const bool ok = idx < kTok * kWgCols && t0 + tt < n && blockIdx.z * kWgCols + cc < g.dv;
      fv[e] = ok ? ldf<T>(pv, (int64_t)(r0 + t0 + tt) * g.vs + cc) : 0.f;
    }
  };
  fetch(0);
  float* outp = g.out + (int64_t)r0 * g.H * g.dv + h * g.dv + j0;
  const bool out4 = g.dv % 4 == 0 && j0 + kCols <= g.dv;
  for (int t0 = 0; t0 < n; t0 += kTok) {
    __syncthreads();  // the previous block's tokens are consumed
#pragma unroll
    for (int e = 0; e < kE; ++e) {
      const int idx = tid + e * NT, tt = idx / kDkp, ch = idx % kDkp;
      if (idx < kTok * kDkp) {
        sr[tt][ch] = fr[e];
        sk[tt][ch] = fk[e];
        su[tt][ch] = fu[e];
        sw[tt][ch] = fw[e];
        sa[tt][ch] = fa[e];
      }
    }
#pragma unroll
    for (int e = 0; e < kEv; ++e) {
      const int idx = tid + e * NT;
      if (idx < kTok * kWgCols) sv[idx / kWgCols][idx % kWgCols] = fv[e];
    }
    __syncthreads();
    if (t0 + kTok < n) fetch(t0 + kTok);
    const int nt = n - t0 < kTok ? n - t0 : kTok;
    // the five row vectors of a token (unit key, decay, removal, key, read-out) and its values
    auto load = [&](int tt, float (*b)[kRows], float* vj) {
#pragma unroll
      for (int q = 0; q < kRows; q += 4) {
        *reinterpret_cast<f32x4*>(b[0] + q) = *reinterpret_cast<const f32x4*>(&su[tt][rq[q / 4]]);
        *reinterpret_cast<f32x4*>(b[1] + q) = *reinterpret_cast<const f32x4*>(&sw[tt][rq[q / 4]]);
        *reinterpret_cast<f32x4*>(b[2] + q) = *reinterpret_cast<const f32x4*>(&sa[tt][rq[q / 4]]);
        *reinterpret_cast<f32x4*>(b[3] + q) = *reinterpret_cast<const f32x4*>(&sk[tt][rq[q / 4]]);
        *reinterpret_cast<f32x4*>(b[4] + q) = *reinterpret_cast<const f32x4*>(&sr[tt][rq[q / 4]]);
      }
#pragma unroll
      for (int c = 0; c < kCols; ++c) vj[c] = sv[tt][grp * kCols + c];
    };
    auto step = [&](const float (*b)[kRows], const float* vj, float* o_) {
      float us[kCols];
#pragma unroll
      for (int c = 0; c < kCols; ++c) {
        float a_ = 0.f;
#pragma unroll
        for (int q = 0; q < kRows; ++q) a_ += b[0][q] * S[c][q];
        us[c] = group_sum<R>(a_);
      }
#pragma unroll
      for (int c = 0; c < kCols; ++c) {
        float a_ = 0.f;
#pragma unroll
        for (int q = 0; q < kRows; ++q) {
          S[c][q] = S[c][q] * b[1][q] - b[2][q] * us[c] + b[3][q] * vj[c];
          a_ += b[4][q] * S[c][q];
        }
        o_[c] = group_sum<R>(a_);
      }
    };
    auto store = [&](int tt, const float* o_) {
      float* op = outp + (int64_t)(t0 + tt) * g.H * g.dv;
      if constexpr (kCols == 4) {
        if (out4) *reinterpret_cast<f32x4*>(op) = f32x4{o_[0], o_[1], o_[2], o_[3]};
      }
      if (kCols != 4 || !out4) {
#pragma unroll
        for (int c = 0; c < kCols; ++c)
          if (j0 + c < g.dv) op[c] = o_[c];
      }
    };
    if (kCols <= 2 && nt == kTok) {
      // a whole block of the narrow tile (the wide one has no registers to spare), unrolled in one basic
      // block: the next token's vectors are read from LDS while the current token's chain runs, and the
      // outputs are stored once at the end
      float b0[5][kRows], b1[5][kRows], v0[kCols], v1[kCols], ob[kTok][kCols];
      load(0, b0, v0);
#pragma unroll
      for (int tt = 0; tt < kTok; tt += 2) {
        load(tt + 1, b1, v1);
        step(b0, v0, ob[tt]);
        if (tt + 2 < kTok) load(tt + 2, b0, v0);
        step(b1, v1, ob[tt + 1]);
      }
      if (part == 0) {
#pragma unroll
        for (int tt = 0; tt < kTok; ++tt) store(tt, ob[tt]);
      }
    } else {
      for (int tt = 0; tt < nt; ++tt) {
        float b0[5][kRows], v0[kCols], o_[kCols];
        load(tt, b0, v0);
        step(b0, v0, o_);
        if (part == 0) store(tt, o_);
      }
    }
  }
#pragma unroll
  for (int c = 0; c < kCols; ++c) {
    if (j0 + c >= g.dv) continue;
    float* spc = sp + (int64_t)(j0 + c) * g.dk;
#pragma unroll
    for (int m = 0; m < kRows / 4; ++m) {
      if (g.dk % 4 == 0 && rq[m] + 4 <= g.dk) {
        *reinterpret_cast<f32x4*>(spc + rq[m]) = f32x4{S[c][4 * m], S[c][4 * m + 1], S[c][4 * m + 2], S[c][4 * m + 3]};
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (rq[m] + e < g.dk) spc[rq[m] + e] = S[c][4 * m + e];
      }
    }
  }
}

// NT threads per workgroup: 64 where that covers all columns of a head, else 256.  Columns per
// thread: the widest tile that still gives the launch two waves per SIMD (2048 on the chip) -- a
// token's chain leaves a lone wave waiting most of the time -- down to one column for a few long prompts.
template <typename T, int R, int CT>
void launch_delta_ct(const DeltaArgs& g, int n_seq, hipStream_t st) {
  const int need = R * ((g.dv + CT - 1) / CT);
  if constexpr (R < 16) {  // (a single wave staging 256 key channels would spill its registers)
    if (need <= 64) {
      hipLaunchKernelGGL((delta_rule_kernel<T, R, 64, CT>), dim3(n_seq, g.H, 1), dim3(64), 0, st, g);
      return;
    }
  }
  {
    const int cols = 256 / R * CT;
    hipLaunchKernelGGL((delta_rule_kernel<T, R, 256, CT>), dim3(n_seq, g.H, (g.dv + cols - 1) / cols), dim3(256), 0,
                       st, g);
  }
}
template <typename T, int R>
void launch_delta(const DeltaArgs& g, int n_seq, hipStream_t st) {
  const int64_t waves4 = (int64_t)n_seq * g.H * ((R * ((g.dv + 3) / 4) + 63) / 64);
  if (waves4 >= 2048) launch_delta_ct<T, R, 4>(g, n_seq, st);
  else if (waves4 >= 1024) launch_delta_ct<T, R, 2>(g, n_seq, st);
  else launch_delta_ct<T, R, 1>(g, n_seq, st);
}

// ---------------------------------------------------------------------------
// Retention: linear attention with one fixed decay per head, no softmax and no
// denominator.  Per (sequence, head) a matrix S [dk, dv]:
//     S_t = decay_h S_(t-1) + (k_scale k_t) v_t^T,   o_t = S_t^T q_t.
// Columns of S are independent: R neighbouring lanes share a column (lane r of
// the group owns rows r, r + R, ..., up to kRows of them, in registers) and join
// their partial q^T S by DPP lane exchanges; a workgroup owns blockDim / R
// columns of one (sequence, head).  Tokens are staged through LDS kTok at a
// time (q, scaled k: [kTok][dk]; v: [kTok][columns]).  State layout as for the
// delta rule: [slots, H, dv, dk], a column's rows contiguous.
struct RetArgs {
  float* out;    // [T, H * dv]
  float* state;  // [slots, H, dv, dk]
  const void *q, *k, *v;
  int64_t qs, ks, vs;  // row strides (elements)
  const float* decay;  // [H]
  float k_scale;
  const int64_t* pos;
  const int* seq_rows;  // null: row i is sequence i
  const int* slots;
  int n_slots, T, H, dk, dv;
};

template <typename T, int R>
__global__ void __launch_bounds__(256) retention_kernel(RetArgs g) {
  extern __shared__ float ret_lds[];
  const int s = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, cols = blockDim.x / R;
  const int cl = tid / R, r = tid % R;
  const int col0 = blockIdx.z * cols, j = col0 + cl;
  const int r0 = g.seq_rows ? g.seq_rows[s] : s, r1 = g.seq_rows ? g.seq_rows[s + 1] : s + 1;
  if (r1 <= r0 || r0 < 0 || r1 > g.T) return;
  const bool colok = j < g.dv;
  const int slot = g.slots[s];
  const int64_t ow = (int64_t)g.H * g.dv;
  if (slot < 0 || slot >= g.n_slots) {  // a padding row: zeros out, no state touched
    for (int t = r0; t < r1; ++t)
      if (r == 0 && colok) g.out[(int64_t)t * ow + h * g.dv + j] = 0.f;
    return;
  }
  float* qs_ = ret_lds;
  float* ks_ = qs_ + kTok * g.dk;
  float* vs_ = ks_ + kTok * g.dk;
  float* sp = g.state + (((int64_t)slot * g.H + h) * g.dv + (colok ? j : 0)) * g.dk;
  const bool fresh = g.pos[r0] == 0;
  float S[kRows];
#pragma unroll
  for (int ii = 0; ii < kRows; ++ii) {
    const int i = r + R * ii;
    S[ii] = (!fresh && colok && i < g.dk) ? sp[i] : 0.f;
  }
  const float dec = g.decay[h];
  const T* q = (const T*)g.q;
  const T* k = (const T*)g.k;
  const T* v = (const T*)g.v;
  for (int t0 = r0; t0 < r1; t0 += kTok) {
    const int nt = r1 - t0 < kTok ? r1 - t0 : kTok;
    __syncthreads();  // the previous block's reads are done
    for (int e = tid; e < nt * g.dk; e += blockDim.x) {
      const int tt = e / g.dk, i = e - tt * g.dk;
      qs_[e] = ldf<T>(q, (int64_t)(t0 + tt) * g.qs + h * g.dk + i);
      ks_[e] = ldf<T>(k, (int64_t)(t0 + tt) * g.ks + h * g.dk + i) * g.k_scale;
    }
    for (int e = tid; e < nt * cols; e += blockDim.x) {
      const int tt = e / cols, c = e - tt * cols;
      vs_[e] = col0 + c < g.dv ? ldf<T>(v, (int64_t)(t0 + tt) * g.vs + h * g.dv + col0 + c) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = vs_[tt * cols + cl];
      const float* qt = qs_ + tt * g.dk;
      const float* kt = ks_ + tt * g.dk;
      float acc = 0.f;
#pragma unroll
      for (int ii = 0; ii < kRows; ++ii) {
        const int i = r + R * ii;
        if (i < g.dk) {
          S[ii] = dec * S[ii] + kt[i] * vj;
          acc += qt[i] * S[ii];
        }
      }
      acc = group_sum<R>(acc);
      if (r == 0 && colok) g.out[(int64_t)(t0 + tt) * ow + h * g.dv + j] = acc;
    }
  }
  if (colok) {
#pragma unroll
    for (int ii = 0; ii < kRows; ++ii) {
      const int i = r + R * ii;
      if (i < g.dk) sp[i] = S[ii];
    }
  }
}

// The same for key widths dk = 16 R and 16-byte aligned operands: nothing in the token loop is
// conditional.  Lane r of a column's group owns the four row quads 4 (r + R qd) .. + 3, qd < 4, so
// a group's 128-bit LDS reads of a q or k row are neighbouring chunks and the state is read and
// written as 16-byte runs.  The next block's eight tokens (q, k of the head, v of the workgroup's
// columns) are fetched into registers as 16-byte chunks while the current block's chain runs.
typedef uint32_t ret_u32x4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ void chunk_to_f32(const ret_u32x4& c, float* o);
template <> __device__ __forceinline__ void chunk_to_f32<bf16_t>(const ret_u32x4& c, float* o) {
#pragma unroll
  for (int i = 0; i < 4; ++i) o[2 * i] = bf16lo(c[i]), o[2 * i + 1] = bf16hi(c[i]);
}
template <> __device__ __forceinline__ void chunk_to_f32<float>(const ret_u32x4& c, float* o) {
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = __uint_as_float(c[i]);
}

template <typename T, int R>
__global__ void __launch_bounds__(256) retention_fast_kernel(RetArgs g) {
  constexpr int dk = 16 * R, cols = 256 / R, VEC = 16 / (int)sizeof(T);
  constexpr int QC = dk / VEC, VC = cols / VEC;          // chunks per token row
  constexpr int QK_CH = kTok * QC, V_CH = kTok * VC, N_CH = 2 * QK_CH + V_CH;
  constexpr int PER = (N_CH + 255) / 256;
  __shared__ __attribute__((aligned(16))) float qs_[kTok * dk];
  __shared__ __attribute__((aligned(16))) float ks_[kTok * dk];
  __shared__ __attribute__((aligned(16))) float vs_[kTok * cols];
  const int s = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, cl = tid / R, r = tid % R;
  const int col0 = blockIdx.z * cols, j = col0 + cl;
  const int r0 = g.seq_rows ? g.seq_rows[s] : s, r1 = g.seq_rows ? g.seq_rows[s + 1] : s + 1;
  if (r1 <= r0 || r0 < 0 || r1 > g.T) return;
  const int slot = g.slots[s];
  const int64_t ow = (int64_t)g.H * g.dv;
  if (slot < 0 || slot >= g.n_slots) {  // a padding row: zeros out, no state touched
    for (int t = r0; t < r1; ++t)
      if (r == 0) g.out[(int64_t)t * ow + h * g.dv + j] = 0.f;
    return;
  }
  float* sp = g.state + (((int64_t)slot * g.H + h) * g.dv + j) * dk;
  const bool fresh = g.pos[r0] == 0;
  float S[16];
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    const f32x4 v4 = fresh ? f32x4{0.f, 0.f, 0.f, 0.f} : *reinterpret_cast<const f32x4*>(sp + 4 * (r + R * qd));
#pragma unroll
    for (int e = 0; e < 4; ++e) S[4 * qd + e] = v4[e];
  }
  const float dec = g.decay[h];
  const T* q = (const T*)g.q + (int64_t)h * dk;
  const T* k = (const T*)g.k + (int64_t)h * dk;
  const T* v = (const T*)g.v + (int64_t)h * g.dv + col0;
  ret_u32x4 pf[PER];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int c = tid + i * 256;
      const T* src = nullptr;
      if (c < QK_CH) {
        const int tt = c / QC;
        if (t0 + tt < r1) src = q + (int64_t)(t0 + tt) * g.qs + (c % QC) * VEC;
      } else if (c < 2 * QK_CH) {
        const int c2 = c - QK_CH, tt = c2 / QC;
        if (t0 + tt < r1) src = k + (int64_t)(t0 + tt) * g.ks + (c2 % QC) * VEC;
      } else if (c < N_CH) {
        const int c2 = c - 2 * QK_CH, tt = c2 / VC;
        if (t0 + tt < r1) src = v + (int64_t)(t0 + tt) * g.vs + (c2 % VC) * VEC;
      }
      pf[i] = src ? *reinterpret_cast<const ret_u32x4*>(src) : ret_u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int c = tid + i * 256;
      float f[VEC];
      chunk_to_f32<T>(pf[i], f);
      float* dst = nullptr;
      if (c < QK_CH) {
        dst = qs_ + c * VEC;
      } else if (c < 2 * QK_CH) {
        dst = ks_ + (c - QK_CH) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) f[e] *= g.k_scale;
      } else if (c < N_CH) {
        dst = vs_ + (c - 2 * QK_CH) * VEC;
      }
      if (dst) {
#pragma unroll
        for (int e = 0; e < VEC; e += 4) *reinterpret_cast<f32x4*>(dst + e) = f32x4{f[e], f[e + 1], f[e + 2], f[e + 3]};
      }
    }
  };
  fetch(r0);
  for (int t0 = r0; t0 < r1; t0 += kTok) {
    const int nt = r1 - t0 < kTok ? r1 - t0 : kTok;
    __syncthreads();  // the previous block's reads are done
    commit();
    __syncthreads();
    if (t0 + kTok < r1) fetch(t0 + kTok);
    for (int tt = 0; tt < nt; ++tt) {
      const float vj = vs_[tt * cols + cl];
      float acc = 0.f;
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const f32x4 kk = *reinterpret_cast<const f32x4*>(ks_ + tt * dk + 4 * (r + R * qd));
        const f32x4 qq = *reinterpret_cast<const f32x4*>(qs_ + tt * dk + 4 * (r + R * qd));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[4 * qd + e] = dec * S[4 * qd + e] + kk[e] * vj;
          acc += qq[e] * S[4 * qd + e];
        }
      }
      acc = group_sum<R>(acc);
      if (r == 0) g.out[(int64_t)(t0 + tt) * ow + h * g.dv + j] = acc;
    }
  }
#pragma unroll
  for (int qd = 0; qd < 4; ++qd)
    *reinterpret_cast<f32x4*>(sp + 4 * (r + R * qd)) = f32x4{S[4 * qd], S[4 * qd + 1], S[4 * qd + 2], S[4 * qd + 3]};
}

// whether the unconditional kernel serves the launch: dk = 16 R exactly, whole column blocks,
// 16-byte aligned rows and sections
template <typename T, int R>
bool retention_fast_ok(const RetArgs& g) {
  constexpr int VEC = 16 / (int)sizeof(T), cols = 256 / R;
  auto al = [](const void* p) { return (uintptr_t)p % 16 == 0; };
  return g.dk == 16 * R && g.dv % cols == 0 && cols % VEC == 0 && g.qs % VEC == 0 && g.ks % VEC == 0 &&
         g.vs % VEC == 0 && al(g.q) && al(g.k) && al(g.v) && al(g.state);
}

template <typename T, int R>
void launch_retention(const RetArgs& g, int n_seq, hipStream_t st) {
  if (retention_fast_ok<T, R>(g)) {
    hipLaunchKernelGGL((retention_fast_kernel<T, R>), dim3(n_seq, g.H, g.dv / (256 / R)), dim3(256), 0, st, g);
    return;
  }

  int nt = (R * g.dv + 63) / 64 * 64;
  nt = nt > 256 ? 256 : nt;
  const int cols = nt / R;
  const size_t lds = (size_t)(2 * kTok * g.dk + kTok * cols) * sizeof(float);
  hipLaunchKernelGGL((retention_kernel<T, R>), dim3(n_seq, g.H, (g.dv + cols - 1) / cols), dim3(nt), lds, st, g);
}

// ---------------------------------------------------------------------------
// Short causal convolution over time on the leading C = n_q d + n_k (d + dv)
// columns of a fused projection, then rotary positions on the first 2 * half
// columns of every q and k head (column i paired with i + half), q to its own
// tensor, k and v into the paged caches.  y_t = sum_j cw[j][c] u_(t - taps + 1 + j);
// u at positions before the step's first row of the sequence comes from the
// sequence's tail state [taps - 1, C], and is zero before position 0.
struct ConvArgs {
  void* q_out;  // [T, n_q * d]
  const void* x;
  int64_t xs;
  const float* cw;  // [taps, C] (tap-major: a run of channels shares a load)
  int taps;
  const void* tail;  // [slots, taps - 1, C]
  int n_slots;
  const int64_t* pos;
  const int64_t* kv_slots;
  const int* row_seq;   // null (with seq_rows null): row i is sequence i
  const int* seq_rows;
  const int* slots;
  int n_seq, T, n_q, n_k, d, dv;
  const float* inv_freq;  // [half]
  int half;
  void* kc;
  void* vc;
};

template <typename T>
__global__ void __launch_bounds__(256) conv_rope_cache_kernel(ConvArgs g) {
  const int t = blockIdx.x;
  const int C = g.n_q * g.d + g.n_k * (g.d + g.dv);
  const int s = g.row_seq ? g.row_seq[t] : t;
  const bool seq_ok = s >= 0 && s < g.n_seq;
  const int r0 = !seq_ok ? t : (g.seq_rows ? g.seq_rows[s] : t);
  const int slot = seq_ok ? g.slots[s] : -1;
  const bool live = slot >= 0 && slot < g.n_slots && r0 >= 0 && r0 <= t;
  const int64_t p = g.pos[t];
  const int64_t p0 = p - (t - r0);  // position of the step's first row of this sequence
  const int m = g.taps - 1;
  const T* x = (const T*)g.x;
  const T* tail = (const T*)g.tail + (int64_t)(live ? slot : 0) * m * C;
  auto conv = [&](int c) -> float {
    float y = 0.f;
    for (int jj = 0; jj < g.taps; ++jj) {
      const int64_t qp = p - m + jj;
      float u = 0.f;
      if (qp >= p0) u = ldf<T>(x, (int64_t)(r0 + (qp - p0)) * g.xs + c);
      else if (qp >= 0) u = ldf<T>(tail, (qp - p0 + m) * C + c);
      y += g.cw[(int64_t)jj * C + c] * u;
    }
    return y;
  };
  // the row's angles: one cosine and sine per rotated pair, shared by all heads
  extern __shared__ float cs_sn[];  // [half] cosines, [half] sines
  for (int i = threadIdx.x; i < g.half; i += blockDim.x) sincosf((float)p * g.inv_freq[i], &cs_sn[g.half + i], &cs_sn[i]);
  __syncthreads();
  const int qk = (g.n_q + g.n_k) * g.d;
  const int64_t kvs = g.kv_slots[t];
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float y = live ? conv(c) : 0.f;
    if (c < qk) {
      const int e = c % g.d;
      if (live && e < 2 * g.half) {
        const int i = e < g.half ? e : e - g.half;
        const float other = conv(e < g.half ? c + g.half : c - g.half);
        const float cs = cs_sn[i], sn = cs_sn[g.half + i];
        y = e < g.half ? y * cs - other * sn : y * cs + other * sn;
      }
      if (c < g.n_q * g.d) stf<T>((T*)g.q_out, (int64_t)t * g.n_q * g.d + c, y);
      else if (kvs >= 0 && live) stf<T>((T*)g.kc, kvs * (g.n_k * g.d) + (c - g.n_q * g.d), y);
    } else if (kvs >= 0 && live) {
      stf<T>((T*)g.vc, kvs * (g.n_k * g.dv) + (c - qk), y);
    }
  }
}

// The same on V consecutive channels per thread with 16-byte loads and stores (V = 8 bf16 or
// 4 fp32): a thread takes a run of the low rotary half together with its partner run of the
// high half, so every channel is convolved once and every angle evaluated once.  Needs d, dv,
// half, the row stride and the cache widths to be multiples of V, and 16-byte aligned bases.
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

// A workgroup takes kConvRows consecutive rows of the step (they may belong to different
// sequences); the taps loop is outermost, so a thread loads a tap's weights once for all its rows.
constexpr int kConvRows = 4;
template <typename T, int V>
__global__ void __launch_bounds__(128) conv_rope_cache_vec_kernel(ConvArgs g) {
  const int t0 = blockIdx.x * kConvRows;
  const int C = g.n_q * g.d + g.n_k * (g.d + g.dv);
  const int m = g.taps - 1;
  const T* x = (const T*)g.x;
  // per row: liveness, position, first position of its sequence in the step, first row, tail, cache slot
  bool live[kConvRows];
  int64_t p[kConvRows], p0[kConvRows], kvs[kConvRows];
  int r0[kConvRows];
  const T* tail[kConvRows];
#pragma unroll
  for (int r = 0; r < kConvRows; ++r) {
    const int t = t0 + r < g.T ? t0 + r : g.T - 1;
    const int s = g.row_seq ? g.row_seq[t] : t;
    const bool seq_ok = s >= 0 && s < g.n_seq;
    r0[r] = !seq_ok ? t : (g.seq_rows ? g.seq_rows[s] : t);
    const int slot = seq_ok ? g.slots[s] : -1;
    live[r] = t0 + r < g.T && slot >= 0 && slot < g.n_slots && r0[r] >= 0 && r0[r] <= t;
    p[r] = g.pos[t];
    p0[r] = p[r] - (t - r0[r]);
    tail[r] = (const T*)g.tail + (int64_t)(live[r] ? slot : 0) * m * C;
    kvs[r] = live[r] ? g.kv_slots[t] : -1;
  }
  extern __shared__ float cs_sn[];  // per row [half] cosines, [half] sines of its angles
  for (int i = threadIdx.x; i < kConvRows * g.half; i += blockDim.x) {
    const int r = i / g.half, e = i - r * g.half;
    sincosf((float)p[r] * g.inv_freq[e], &cs_sn[(2 * r + 1) * g.half + e], &cs_sn[2 * r * g.half + e]);
  }
  __syncthreads();
  const int qk = (g.n_q + g.n_k) * g.d, nq = g.n_q * g.d;
  auto put = [&](int r, int c, const float* y) {
    if (t0 + r >= g.T) return;
    if (c < nq) VecIO<T, V>::st((T*)g.q_out + (int64_t)(t0 + r) * nq + c, y);
    else if (kvs[r] < 0) return;
    else if (c < qk) VecIO<T, V>::st((T*)g.kc + kvs[r] * (g.n_k * g.d) + (c - nq), y);
    else VecIO<T, V>::st((T*)g.vc + kvs[r] * (g.n_k * g.dv) + (c - qk), y);
  };
  // work items: per q / k head its rotated pairs of runs (a run of the low half with its partner of
  // the high half), then its runs that are not rotated; then the runs of v
  const int n_pair = g.half / V, per_head = n_pair + (g.d - 2 * g.half) / V;
  const int n_head_items = (g.n_q + g.n_k) * per_head, n_items = n_head_items + (C - qk) / V;
  for (int it = threadIdx.x; it < n_items; it += blockDim.x) {
    int c, e;
    bool pair = false;
    if (it < n_head_items) {
      const int hd = it / per_head, j = it - hd * per_head;
      pair = j < n_pair;
      e = pair ? j * V : 2 * g.half + (j - n_pair) * V;
      c = hd * g.d + e;
    } else {
      e = 0;
      c = qk + (it - n_head_items) * V;
    }
    float y[kConvRows][V], z[kConvRows][V];
#pragma unroll
    for (int r = 0; r < kConvRows; ++r)
#pragma unroll
      for (int i = 0; i < V; ++i) y[r][i] = z[r][i] = 0.f;
    for (int jj = 0; jj < g.taps; ++jj) {
      float w[V], w2[V];
      const float* wp = g.cw + (int64_t)jj * C + c;
#pragma unroll
      for (int i = 0; i < V; i += 4) *reinterpret_cast<f32x4*>(w + i) = *reinterpret_cast<const f32x4*>(wp + i);
      if (pair) {
#pragma unroll
        for (int i = 0; i < V; i += 4)
          *reinterpret_cast<f32x4*>(w2 + i) = *reinterpret_cast<const f32x4*>(wp + g.half + i);
      }
#pragma unroll
      for (int r = 0; r < kConvRows; ++r) {
        const int64_t qp = p[r] - m + jj;
        if (!live[r] || qp < 0) continue;
        const T* src = qp >= p0[r] ? x + (int64_t)(r0[r] + (qp - p0[r])) * g.xs + c : tail[r] + (qp - p0[r] + m) * C + c;
        float u[V];
        VecIO<T, V>::ld(src, u);
#pragma unroll
        for (int i = 0; i < V; ++i) y[r][i] += w[i] * u[i];
        if (pair) {
          VecIO<T, V>::ld(src + g.half, u);
#pragma unroll
          for (int i = 0; i < V; ++i) z[r][i] += w2[i] * u[i];
        }
      }
    }
#pragma unroll
    for (int r = 0; r < kConvRows; ++r) {
      if (pair) {
        float lo[V], hi[V];
        const float* cs = cs_sn + 2 * r * g.half + e;
        const float* sn = cs + g.half;
#pragma unroll
        for (int i = 0; i < V; ++i) {
          lo[i] = y[r][i] * cs[i] - z[r][i] * sn[i];
          hi[i] = z[r][i] * cs[i] + y[r][i] * sn[i];
        }
        put(r, c, lo);
        put(r, c + g.half, hi);
      } else {
        put(r, c, y[r]);
      }
    }
  }
}

// tail [slots, m, C] <- the last m projected rows of every sequence of the step
template <typename T>
__global__ void __launch_bounds__(256) conv_state_update_kernel(T* __restrict__ tail, int n_slots,
                                                                const T* __restrict__ x, int64_t xs,
                                                                const int64_t* __restrict__ pos,
                                                                const int* __restrict__ seq_rows,
                                                                const int* __restrict__ slots, int T_, int C, int m) {
  const int s = blockIdx.x;
  const int r0 = seq_rows ? seq_rows[s] : s, r1 = seq_rows ? seq_rows[s + 1] : s + 1;
  const int slot = slots[s];
  const int n = r1 - r0;
  if (slot < 0 || slot >= n_slots || n <= 0 || r0 < 0 || r1 > T_) return;
  const int64_t p0 = pos[r0];
  T* ts = tail + (int64_t)slot * m * C;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
    // new[i] is the step-relative row n - m + i: a row of x, or an old entry shifted down.
    // Ascending i reads old entries at i + n > i only, so a thread may overwrite as it goes.
    for (int i = 0; i < m; ++i) {
      const int rel = n - m + i;
      T val;
      if (rel >= 0) val = x[(int64_t)(r0 + rel) * xs + c];
      else if (p0 + rel >= 0) val = ts[(int64_t)(i + n) * C + c];
      else val = (T)0;
      ts[(int64_t)i * C + c] = val;
    }
  }
}

// out = o / sqrt(mean_head(o^2) + eps) * w * sigmoid(gate) (or * silu(gate)): one wave per (row, head), four per workgroup;
// a lane keeps its elements (V neighbours at a time, up to kHnKeep times) in registers between the mean
// square and the result.  V = 2 needs an even dv and gate stride and 8-byte aligned o and w.
constexpr int kHnKeep = 4;
template <typename T, int V>
__global__ void __launch_bounds__(256) head_norm_gate_kernel(T* __restrict__ out, const float* __restrict__ o,
                                                             const float* __restrict__ w, const T* __restrict__ gate,
                                                             int64_t gs, int64_t n_vec, int H, int dv, float eps,
                                                             int gate_act) {
  const int lane = threadIdx.x & 63;
  const int64_t v = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (v >= n_vec) return;
  const int64_t row = v / H;
  const int h = (int)(v - row * H);
  const float* op = o + v * dv;
  auto ldo = [&](int e, float* x) {
    if constexpr (V == 2) {
      const float2 t = *reinterpret_cast<const float2*>(op + e);
      x[0] = t.x, x[1] = t.y;
    } else {
      x[0] = op[e];
    }
  };
  float x[kHnKeep][V], ss = 0.f;
#pragma unroll
  for (int k = 0; k < kHnKeep; ++k) {
    const int e = (lane + 64 * k) * V;
#pragma unroll
    for (int i = 0; i < V; ++i) x[k][i] = 0.f;
    if (e < dv) ldo(e, x[k]);
#pragma unroll
    for (int i = 0; i < V; ++i) ss += x[k][i] * x[k][i];
  }
  for (int e = (lane + 64 * kHnKeep) * V; e < dv; e += 64 * V) {
    float t[V];
    ldo(e, t);
#pragma unroll
    for (int i = 0; i < V; ++i) ss += t[i] * t[i];
  }
  const float inv = rsqrtf(wave_reduce_sum(ss) / (float)dv + eps);
  auto put = [&](int e, const float* xv) {
    float y[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      y[i] = xv[i] * inv;
      if (w) y[i] *= w[h * dv + e + i];
      if (gate) {  // gate_act 0: sigmoid(z); 1: silu, z sigmoid(z)
        const float z = ldf<T>(gate, row * gs + h * dv + e + i);
        y[i] *= gate_act ? z * sigmoidf_(z) : sigmoidf_(z);
      }
    }
    if constexpr (V == 2 && sizeof(T) == 2) {
      *reinterpret_cast<uint32_t*>((bf16_t*)out + v * dv + e) = pack_bf16x2(y[0], y[1]);
    } else {
#pragma unroll
      for (int i = 0; i < V; ++i) stf<T>(out, v * dv + e + i, y[i]);
    }
  };
#pragma unroll
  for (int k = 0; k < kHnKeep; ++k)
    if ((lane + 64 * k) * V < dv) put((lane + 64 * k) * V, x[k]);
  for (int e = (lane + 64 * kHnKeep) * V; e < dv; e += 64 * V) {
    float t[V];
    ldo(e, t);
    put(e, t);
  }
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

int dxm_delta_rule(float* out, float* state, int n_slots, float* prep, const void* r, int64_t rs, const void* k,
                   int64_t ks, const void* v, int64_t vs, const void* a, int64_t as, const void* w, int64_t ws,
                   const float* a_bias, const float* w_bias, float decay_scale, float key_eps, const int64_t* pos,
                   const int* seq_rows, const int* slots, int n_seq, int T_, int H, int dk, int dv, int f32,
                   hipStream_t st) {
  if (n_seq <= 0 || T_ <= 0) return 0;
  if (H < 1 || dk < 1 || dv < 1 || n_slots < 1 || H > 65535 || n_seq > 0x7fffffff || (int64_t)T_ * H > 0x7fffffff)
    return 1;
  if (dk > kRows * 16) return 2;  // wider keys need more lanes per column than instantiated
  if (!out || !state || !pos || !slots || !prep) return 3;
  if (!seq_rows && n_seq != T_) return 4;
  DISPATCH_T(f32, hipLaunchKernelGGL(delta_prep_kernel<T>, dim3((unsigned)(T_ * H)), dim3(64), 0, st, prep, (const T*)k,
                                     ks, (const T*)a, as, (const T*)w, ws, a_bias, w_bias, decay_scale, key_eps, H, dk));
  DeltaArgs g{out, state, r, k, v, rs, ks, vs, prep, pos, seq_rows, slots, n_slots, T_, H, dk, dv};
  const int need = (dk + kRows - 1) / kRows;
  if (need <= 4) { DISPATCH_T(f32, (launch_delta<T, 4>(g, n_seq, st))); }
  else if (need <= 8) { DISPATCH_T(f32, (launch_delta<T, 8>(g, n_seq, st))); }
  else { DISPATCH_T(f32, (launch_delta<T, 16>(g, n_seq, st))); }
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_retention(float* out, float* state, int n_slots, const void* q, int64_t qs, const void* k, int64_t ks,
                  const void* v, int64_t vs, const float* decay, float k_scale, const int64_t* pos,
                  const int* seq_rows, const int* slots, int n_seq, int T_, int H, int dk, int dv, int f32,
                  hipStream_t st) {
  if (n_seq <= 0 || T_ <= 0) return 0;
  if (H < 1 || dk < 1 || dv < 1 || n_slots < 1 || H > 65535 || (int64_t)T_ * H * dv > 0x7fffffffffffLL) return 1;
  if (dk > kRows * 16) return 2;  // wider keys need more lanes per column than instantiated
  if (!out || !state || !pos || !slots || !decay || !q || !k || !v) return 3;
  if (!seq_rows && n_seq != T_) return 4;
  RetArgs g{out, state, q, k, v, qs, ks, vs, decay, k_scale, pos, seq_rows, slots, n_slots, T_, H, dk, dv};
  const int need = (dk + kRows - 1) / kRows;
  if (need <= 1) { DISPATCH_T(f32, (launch_retention<T, 1>(g, n_seq, st))); }
  else if (need <= 2) { DISPATCH_T(f32, (launch_retention<T, 2>(g, n_seq, st))); }
  else if (need <= 4) { DISPATCH_T(f32, (launch_retention<T, 4>(g, n_seq, st))); }
  else if (need <= 8) { DISPATCH_T(f32, (launch_retention<T, 8>(g, n_seq, st))); }
  else { DISPATCH_T(f32, (launch_retention<T, 16>(g, n_seq, st))); }
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_conv_rope_cache(void* q_out, const void* x, int64_t xs, const float* cw, int taps, const void* tail,
                        int n_slots, const int64_t* pos, const int64_t* kv_slots, const int* row_seq,
                        const int* seq_rows, const int* slots, int n_seq, int T_, int n_q, int n_k, int d, int dv,
                        const float* inv_freq, int half, void* kc, void* vc, int f32, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (taps < 1 || n_q < 0 || n_k < 0 || d < 1 || dv < 0 || half < 0 || 2 * half > d || half > 4096) return 1;
  if ((half && !inv_freq) || (n_k && (!kc || !vc)) || (taps > 1 && !tail) || !cw || !pos || !kv_slots || !slots)
    return 2;
  if ((row_seq == nullptr) != (seq_rows == nullptr) || (!row_seq && n_seq != T_)) return 3;
  ConvArgs g{q_out, x, xs, cw, taps, tail, n_slots, pos, kv_slots, row_seq, seq_rows, slots, n_seq, T_,
             n_q, n_k, d, dv, inv_freq, half, kc, vc};
  const int V = f32 ? 4 : 8, esz = f32 ? 4 : 2;
  auto al = [&](const void* ptr) { return (uintptr_t)ptr % 16 == 0; };
  const bool vec = d % V == 0 && dv % V == 0 && half % V == 0 && xs % V == 0 && al(x) && al(q_out) && al(tail) &&
                   al(kc) && al(vc) && al(cw) && ((n_q * d + n_k * (d + dv)) * esz) % 16 == 0;
  const size_t lds = (size_t)2 * half * sizeof(float);
  const dim3 vgrid((T_ + kConvRows - 1) / kConvRows);
  if (vec && f32) hipLaunchKernelGGL((conv_rope_cache_vec_kernel<float, 4>), vgrid, dim3(128), kConvRows * lds, st, g);
  else if (vec) hipLaunchKernelGGL((conv_rope_cache_vec_kernel<bf16_t, 8>), vgrid, dim3(128), kConvRows * lds, st, g);
  else { DISPATCH_T(f32, hipLaunchKernelGGL(conv_rope_cache_kernel<T>, dim3(T_), dim3(256), lds, st, g)); }
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_conv_state_update(void* tail, int n_slots, const void* x, int64_t xs, const int64_t* pos, const int* seq_rows,
                          const int* slots, int n_seq, int T_, int C, int taps, int f32, hipStream_t st) {
  if (n_seq <= 0 || taps <= 1 || C <= 0) return 0;
  if (!tail || !x || !pos || !slots || (!seq_rows && n_seq != T_)) return 1;
  const int gy = (C + 255) / 256 < 64 ? (C + 255) / 256 : 64;
  DISPATCH_T(f32, hipLaunchKernelGGL(conv_state_update_kernel<T>, dim3(n_seq, gy), dim3(256), 0, st, (T*)tail, n_slots,
                                     (const T*)x, xs, pos, seq_rows, slots, T_, C, taps - 1));
  DX_CHECK_LAUNCH();
  return 0;
}

int dxm_head_norm_gate(void* out, const float* o, const float* w, const void* gate, int64_t gs, int rows, int H,
                       int dv, float eps, int gate_act, int f32, hipStream_t st) {
  if (rows <= 0) return 0;
  if (H < 1 || dv < 1 || (int64_t)rows * H > 0x7fffffff || gate_act < 0 || gate_act > 1) return 1;
  const int64_t n_vec = (int64_t)rows * H;
  const dim3 grid((unsigned)((n_vec + 3) / 4));
  const bool v2 = dv % 2 == 0 && gs % 2 == 0 && (uintptr_t)o % 8 == 0 && (uintptr_t)out % 4 == 0;
  if (v2) {
    DISPATCH_T(f32, hipLaunchKernelGGL((head_norm_gate_kernel<T, 2>), grid, dim3(256), 0, st, (T*)out, o, w,
                                       (const T*)gate, gs, n_vec, H, dv, eps, gate_act));
  } else {
    DISPATCH_T(f32, hipLaunchKernelGGL((head_norm_gate_kernel<T, 1>), grid, dim3(256), 0, st, (T*)out, o, w,
                                       (const T*)gate, gs, n_vec, H, dv, eps, gate_act));
  }
  DX_CHECK_LAUNCH();
  return 0;
}

}  // extern "C"
