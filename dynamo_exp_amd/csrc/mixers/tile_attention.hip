// Paged softmax attention for prompt chunks on the gfx950 matrix cores: the
// prefill kernel of the layer-listed models (bf16 q / caches, head widths that
// are multiples of 16; everything else runs row_attention.hip).
//
// A workgroup (4 waves) takes up to 128 consecutive rows of one sequence and
// one query vector (head x map); a wave owns 32 of the rows as two 16-row
// blocks.  64-key tiles of the paged, token-major caches are staged in LDS (K
// row-major, V transposed) and shared by the four waves.  Both products are
// "swapped" so the query sits on the lane:
//     S^T = K Q^T     A = K rows (LDS), B = Q^T (registers, loaded once)
//     O^T = V^T P^T   A = V^T (LDS),    B = P^T = the S^T accumulator itself
// (v_mfma_f32_16x16x16_bf16: lane l holds column l % 16 and rows 4 (l / 16)
// .. + 3 of C, which is exactly the B layout of the next product).  Scores are
// the exact fp32 sums of bf16 products; the softmax is fp32.  With bf16 output
// the weights enter the second product as bf16, like the other bf16
// activations; with fp32 output (and in the decode kernel) as a bf16 pair
// hi + lo (two MFMAs), which keeps 16 mantissa bits of every weight.
//
// Optional score terms (uniform per launch): a tanh cap, s <- cap tanh(s / cap),
// and a per-head penalty r1 ln(1 + r2 (p - j)) that grows with the logarithm of
// the distance; both are applied per element in fp32 before the softmax, in
// log2 units (tanh from one exp2 and one reciprocal, the logarithm as v_log).
//
// Masks are evaluated per element in sequence positions: causal, sliding
// window (p - size < j <= p; with `keep` > 0 also the sequence's first `keep`
// keys, j < keep) and chunked (floor(j / size) == floor(p / size)), so a prompt
// cut anywhere gives the same result as one cut nowhere.  Key tiles run over
// one numbering u of the keys a row block can see: the kept first nf keys
// (positions 0 .. nf - 1), then the positions from the window's start on
// (position u + shift); without kept keys nf = 0 and u + shift is the position.
// With `sink` (a number per query vector) exp(sink) joins a softmax's
// denominator once: a key without a value, neither scaled nor masked.
#include "../kernels/common.h"

namespace {

constexpr int kRows = 128;  // rows per workgroup
constexpr int kKeys = 64;   // keys per tile
constexpr int kVtStride = kKeys + 8;
// decode rows of wide heads: a narrower pad lets a third one-wave workgroup share a CU's LDS
constexpr int kVtStrideWide = kKeys + 4;

struct TileArgs {
  const bf16_t* q;
  int64_t q_stride;
  const bf16_t* kc;
  const bf16_t* vc;
  void* out;  // [rows, n_qh, dv]
  const int64_t* pos;
  const int* seq;
  const int* bt;
  int bt_stride, bs;
  const int* tiles;  // [n_tiles, 2]: first row, row count (<= 128; one sequence, consecutive positions)
  int n_qh, maps, group;
  int Wk, Wv;
  float scale;
  int mask, size;
  float softcap;    // 0: none
  const float* r1;  // [n_qh], null: no distance penalty
  const float* r2;
  int wfn;             // 0: softmax; 1: sigmoid(s + hbias) per visible key, not normalised
  const float* hbias;  // [n_qh] (sigmoid weights only; a constant per head leaves a softmax unchanged)
  const bf16_t* gate;  // [rows, gate_stride] logits per head: the result is multiplied by their sigmoid
  int64_t gate_stride;
  int keep;           // window mask: the first `keep` keys of a sequence stay visible (0: none)
  const float* sink;  // [n_qh], softmax only (null: none)
};

constexpr float kLog2e = 1.4426950408889634f;

// cap * tanh(s / cap) * log2(e) for s in natural units: tanh(x) = 1 - 2 / (1 + e^(2x))
__device__ __forceinline__ float capped_log2(float s, float cap, float inv_cap) {
  const float e = fast_exp2(s * (2.f * kLog2e) * inv_cap);
  return cap * kLog2e * (1.f - 2.f * __builtin_amdgcn_rcpf(1.f + e));
}

// positions are < 2^31: 32-bit arithmetic in the kernels
__device__ __forceinline__ int first_visible(int p, int mask, int size) {
  if (mask == 1) return p - size + 1 > 0 ? p - size + 1 : 0;
  if (mask == 2) return (int)((unsigned)p / (unsigned)size) * size;
  return 0;
}

// A 64-key tile of one K head and one V head on its way from the paged caches
// to LDS, split in two so the next tile's global loads fly during the current
// tile's MFMAs: fetch() global -> registers, commit() registers -> LDS (K
// row-major [64][d + 8]; V transposed [dv][64 + 8], four keys of one column
// per 8-byte store).  Keys beyond `hi` arrive as zeros.  NT threads; work items
// are 16-byte chunks, consecutive threads on consecutive chunks of a row.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int d, int dv, int NT, int VS = kVtStride>
struct TileStage {
  static constexpr int ks_stride = d + 8;
  static constexpr int kItems = kKeys * (d / 8), vItems = (kKeys / 4) * (dv / 8);
  static constexpr int kPer = (kItems + NT - 1) / NT, vPer = (vItems + NT - 1) / NT;
  u32x4 kr[kPer];
  u32x4 vr[vPer][4];

  // slot of sequence position kj: block-table lookup in 32-bit arithmetic (a shift
  // for the usual power-of-two block sizes; 64-bit divisions here cost more than the loads)
  static __device__ __forceinline__ int64_t slot_of(const int* bt, int bs, int kj) {
    const unsigned u = (unsigned)kj, b = (unsigned)bs;
    if ((b & (b - 1)) == 0) {
      const int sh = __builtin_ctz(b);
      return ((int64_t)bt[u >> sh] << sh) + (u & (b - 1));
    }
    return (int64_t)bt[u / b] * bs + u % b;
  }

  template <bool DoK = true, bool DoV = true>
  __device__ __forceinline__ void fetch(const bf16_t* kc, const bf16_t* vc, const int* bt, int bs, int Wk, int Wv,
                                        int u0, int nf, int shift, int hi, int tid) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    // One block-table lookup per lane (key kt + lane), handed to the lanes that load
    // the key by a cross-lane read: a lookup per 16-byte load would put a dependent
    // global round trip in front of each of them, and the loads retire in order.
    // (key u0 + lane of the visible keys' numbering: position u below nf, u + shift from there on)
    const int ku = u0 + (tid & 63), kp = ku < nf ? ku : ku + shift;
    const int mine = kp <= hi ? (int)slot_of(bt, bs, kp) : -1;
#pragma unroll
    for (int i = 0; i < (DoK ? kPer : 0); ++i) {
      const int it = tid + i * NT;
      const int key = it / (d / 8), ch = it % (d / 8);
      const int64_t slot = __shfl(mine, key & 63, 64);
      const bool ok = it < kItems && slot >= 0;
      kr[i] = ok ? *reinterpret_cast<const u32x4*>(kc + slot * Wk + ch * 8) : zero;
    }
#pragma unroll
    for (int i = 0; i < (DoV ? vPer : 0); ++i) {
      const int it = tid + i * NT;
      const int kg = it / (dv / 8), ch = it % (dv / 8);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int64_t slot = __shfl(mine, (4 * kg + k) & 63, 64);
        const bool ok = it < vItems && slot >= 0;
        vr[i][k] = ok ? *reinterpret_cast<const u32x4*>(vc + slot * Wv + ch * 8) : zero;
      }
    }
  }

  template <bool DoK = true, bool DoV = true>
  __device__ __forceinline__ void commit(bf16_t* Ks, bf16_t* Vt, int tid) const {
#pragma unroll
    for (int i = 0; i < (DoK ? kPer : 0); ++i) {
      const int it = tid + i * NT;
      if (it < kItems) *reinterpret_cast<u32x4*>(Ks + (it / (d / 8)) * ks_stride + (it % (d / 8)) * 8) = kr[i];
    }
#pragma unroll
    for (int i = 0; i < (DoV ? vPer : 0); ++i) {
      const int it = tid + i * NT;
      if (it >= vItems) continue;
      const int kg = it / (dv / 8), ch = it % (dv / 8);
#pragma unroll
      for (int w = 0; w < 4; ++w) {  // columns ch * 8 + 2 w, + 1: the four keys' values side by side
        uint2 lo, hi2;
        lo.x = (vr[i][0][w] & 0xffffu) | (vr[i][1][w] << 16);
        lo.y = (vr[i][2][w] & 0xffffu) | (vr[i][3][w] << 16);
        hi2.x = (vr[i][0][w] >> 16) | (vr[i][1][w] & 0xffff0000u);
        hi2.y = (vr[i][2][w] >> 16) | (vr[i][3][w] & 0xffff0000u);
        *reinterpret_cast<uint2*>(Vt + (ch * 8 + 2 * w) * VS + 4 * kg) = lo;
        *reinterpret_cast<uint2*>(Vt + (ch * 8 + 2 * w + 1) * VS + 4 * kg) = hi2;
      }
    }
  }
};

typedef short i16x8 __attribute__((ext_vector_type(8)));
// two 4-element fragments side by side as one K = 32 MFMA operand: slots 0..3 and
// 4..7 of a lane group may hold any 8 of the 32 reduction indices, as long as
// A and B agree -- here the lane group's 4 keys of two neighbouring 16-key blocks
__device__ __forceinline__ bf16x8_t pair8(i16x4 a, i16x4 b) {
  return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7));
}

template <typename OutT> __device__ __forceinline__ void store4(OutT* o, f32x4 v);
template <> __device__ __forceinline__ void store4<float>(float* o, f32x4 v) { *reinterpret_cast<f32x4*>(o) = v; }
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* o, f32x4 v) {
  uint2 w;
  w.x = pack_bf16x2(v[0], v[1]);
  w.y = pack_bf16x2(v[2], v[3]);
  *reinterpret_cast<uint2*>(o) = w;
}

template <int DB, int DVB, typename OutT>
__global__ void __launch_bounds__(256, (DB + DVB <= 16 ? 2 : 1)) tile_attention_kernel(TileArgs a) {
  constexpr int d = DB * 16, dv = DVB * 16, ks_stride = d + 8;
  // fp32 output (the two-map layers, whose a1 - lambda a2 amplifies errors): the weights enter
  // the second product as hi + lo; bf16 output: as one bf16, like every other bf16 activation
  constexpr bool kHiLo = sizeof(OutT) == 4;
  constexpr bool X32 = DB % 2 == 0;  // d a multiple of 32: the K = 32 MFMA for the scores too
  constexpr int DB2 = X32 ? DB / 2 : 1;
  extern __shared__ __attribute__((aligned(16))) bf16_t smem[];
  bf16_t* Ks = smem;                    // [64][d + 8]
  bf16_t* Vt = smem + kKeys * ks_stride;  // [dv][64 + 8]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int c16 = lane & 15, g4 = lane >> 4;
  const int qh = blockIdx.x;
  // later tiles of a prompt see more keys: hand them out first (longest first)
  const int ti = gridDim.y - 1 - blockIdx.y;
  const int row0 = a.tiles[2 * ti], n = a.tiles[2 * ti + 1];
  const int p0 = (int)a.pos[row0];
  const int* bt = a.bt + (int64_t)a.seq[row0] * a.bt_stride;
  const int head = qh / a.maps, m = qh - head * a.maps, g = head / a.group;
  const bf16_t* kc = a.kc + (int64_t)(g * a.maps + m) * d;
  const bf16_t* vc = a.vc + (int64_t)g * dv;
  const int hi = p0 + n - 1;
  const int lo0 = first_visible(p0, a.mask, a.size) / kKeys * kKeys;
  const int nf = a.mask == 1 && a.keep > 0 ? (a.keep < lo0 ? a.keep : lo0) : 0;
  const int shift = lo0 - nf, u_end = hi - shift;

  // this wave's query fragments and per-row constants
  i16x4 qf[2][DB];
  bf16x8_t qf8[2][DB2];
  int prow[2], lrow[2];
  bool okrow[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int r = 32 * w + 16 * qb + c16;
    okrow[qb] = r < n;
    prow[qb] = p0 + r;
    lrow[qb] = first_visible(prow[qb], a.mask, a.size);
    const bf16_t* q = a.q + (int64_t)(row0 + (okrow[qb] ? r : 0)) * a.q_stride + (int64_t)qh * d + 4 * g4;
    if constexpr (X32) {
#pragma unroll
      for (int ks = 0; ks < DB2; ++ks)
        qf8[qb][ks] = okrow[qb] ? *reinterpret_cast<const bf16x8_t*>(q + 4 * g4 + ks * 32)
                                : __builtin_bit_cast(bf16x8_t, i16x8{0, 0, 0, 0, 0, 0, 0, 0});
    } else {
#pragma unroll
      for (int ks = 0; ks < DB; ++ks)
        qf[qb][ks] = okrow[qb] ? *reinterpret_cast<const i16x4*>(q + ks * 16) : i16x4{0, 0, 0, 0};
    }
  }
  const bool wave_on = 32 * w < n;
  const bool terms = a.softcap > 0.f || a.r1 != nullptr;
  const float cap = a.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  const float r1 = a.r1 ? a.r1[qh] : 0.f, r2 = a.r1 ? a.r2[qh] : 0.f;
  const float sc2 = terms ? 1.f : a.scale * kLog2e;  // scores in log2 units: exp2 is one instruction
  const float hb2 = a.hbias ? a.hbias[qh] * kLog2e : 0.f;
  float mx[2] = {-INFINITY, -INFINITY}, lsum[2] = {0.f, 0.f};
  f32x4 O[2][DVB];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int cb = 0; cb < DVB; ++cb) O[qb][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

  TileStage<d, dv, 256> stage;
  stage.fetch(kc, vc, bt, a.bs, a.Wk, a.Wv, 0, nf, shift, hi, tid);
  for (int ut = 0; ut <= u_end; ut += kKeys) {
    // a tile that holds both kept first keys and window keys maps its keys one by one
    const bool strad = ut < nf && ut + kKeys > nf;
    const int kt = ut >= nf ? ut + shift : ut;
    auto kpos = [&](int off) { return strad && ut + off >= nf ? kt + off + shift : kt + off; };
    stage.commit(Ks, Vt, tid);
    __syncthreads();
    if (ut + kKeys <= u_end) stage.fetch(kc, vc, bt, a.bs, a.Wk, a.Wv, ut + kKeys, nf, shift, hi, tid);
    if (wave_on) {
      f32x4 S[2][4];
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        S[0][kb] = S[1][kb] = f32x4{0.f, 0.f, 0.f, 0.f};
        if constexpr (X32) {
#pragma unroll
          for (int ks = 0; ks < DB2; ++ks) {
            const bf16x8_t A =
                *reinterpret_cast<const bf16x8_t*>(Ks + (kb * 16 + c16) * ks_stride + ks * 32 + 8 * g4);
            S[0][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A, qf8[0][ks], S[0][kb], 0, 0, 0);
            S[1][kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A, qf8[1][ks], S[1][kb], 0, 0, 0);
          }
        } else {
#pragma unroll
          for (int ks = 0; ks < DB; ++ks) {
            const i16x4 A = *reinterpret_cast<const i16x4*>(Ks + (kb * 16 + c16) * ks_stride + ks * 16 + 4 * g4);
            S[0][kb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(A, qf[0][ks], S[0][kb], 0, 0, 0);
            S[1][kb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(A, qf[1][ks], S[1][kb], 0, 0, 0);
          }
        }
      }
      if (terms) {  // final scores in log2 units; the exponent's multiplier becomes 1
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int kb = 0; kb < 4; ++kb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float s2 = S[qb][kb][i] * a.scale;
              s2 = cap > 0.f ? capped_log2(s2, cap, inv_cap) : s2 * kLog2e;
              if (a.r1) {
                const int dist = prow[qb] - kpos(kb * 16 + 4 * g4 + i);
                s2 -= r1 * __builtin_amdgcn_logf(1.f + r2 * (float)(dist > 0 ? dist : 0));
              }
              S[qb][kb][i] = s2;
            }
      }
      // a tile every row of the wave sees whole needs no per-element mask
      const bool full = 32 * w + 31 < n && !strad && kt + kKeys - 1 <= p0 + 32 * w &&
                        (ut + kKeys <= nf || kt >= first_visible(p0 + 32 * w + 31, a.mask, a.size));
      i16x4 Ph[2][4], Pl[2][4];
      if (a.wfn) {
        // sigmoid weights: w = 1 / (1 + 2^-(x log2 e)), x = s + hbias; invisible keys weigh 0;
        // no maximum, no rescaling, no normalisation
        const float xs = terms ? 1.f : a.scale * kLog2e;
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int kb = 0; kb < 4; ++kb) {
            float p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int kj = kpos(kb * 16 + 4 * g4 + i);
              const bool vis = full || (okrow[qb] && (kj >= lrow[qb] || kj < a.keep) && kj <= prow[qb]);
              const float w_ = __builtin_amdgcn_rcpf(1.f + fast_exp2(-fmaf(S[qb][kb][i], xs, hb2)));
              p[i] = vis ? w_ : 0.f;
            }
            const uint32_t h01 = pack_bf16x2(p[0], p[1]), h23 = pack_bf16x2(p[2], p[3]);
            Ph[qb][kb] = __builtin_bit_cast(i16x4, uint2{h01, h23});
            if constexpr (kHiLo) {
              const uint32_t l01 = pack_bf16x2(p[0] - bf16lo(h01), p[1] - bf16hi(h01));
              const uint32_t l23 = pack_bf16x2(p[2] - bf16lo(h23), p[3] - bf16hi(h23));
              Pl[qb][kb] = __builtin_bit_cast(i16x4, uint2{l01, l23});
            }
          }
      } else {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        // scale > 0 (checked on the host): the row maximum is taken over the raw sums and
        // scaled once, and the scale rides in the exponent's fma
        float mloc = -INFINITY;
        if (full) {
#pragma unroll
          for (int kb = 0; kb < 4; ++kb)
#pragma unroll
            for (int i = 0; i < 4; ++i) mloc = fmaxf(mloc, S[qb][kb][i]);
        } else {
#pragma unroll
          for (int kb = 0; kb < 4; ++kb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int kj = kpos(kb * 16 + 4 * g4 + i);
              const bool vis = okrow[qb] && (kj >= lrow[qb] || kj < a.keep) && kj <= prow[qb];
              const float s = vis ? S[qb][kb][i] : -INFINITY;
              S[qb][kb][i] = s;
              mloc = fmaxf(mloc, s);
            }
        }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
        const float mn = fmaxf(mx[qb], mloc * sc2);  // log2 units
        const float mu = mn == -INFINITY ? 0.f : mn;  // a row that sees nothing in this tile
        const float alpha = fast_exp2(mx[qb] - mu);
        mx[qb] = mn;
        float add = 0.f;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
          float p[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            p[i] = fast_exp2(fmaf(S[qb][kb][i], sc2, -mu));
            add += p[i];
          }
          const uint32_t h01 = pack_bf16x2(p[0], p[1]), h23 = pack_bf16x2(p[2], p[3]);
          Ph[qb][kb] = __builtin_bit_cast(i16x4, uint2{h01, h23});
          if constexpr (kHiLo) {
            const uint32_t l01 = pack_bf16x2(p[0] - bf16lo(h01), p[1] - bf16hi(h01));
            const uint32_t l23 = pack_bf16x2(p[2] - bf16lo(h23), p[3] - bf16hi(h23));
            Pl[qb][kb] = __builtin_bit_cast(i16x4, uint2{l01, l23});
          }
        }
        // the running maximum of no row of the wave moved: nothing to rescale
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
          lsum[qb] = lsum[qb] * alpha + add;
#pragma unroll
          for (int cb = 0; cb < DVB; ++cb) O[qb][cb] *= alpha;
        } else {
          lsum[qb] += add;
        }
      }
      }
#pragma unroll
      for (int kp = 0; kp < 2; ++kp) {  // 32 keys per MFMA: key blocks 2 kp and 2 kp + 1
        bf16x8_t Bh[2], Bl[2];
#pragma unroll
        for (int qb = 0; qb < 2; ++qb) {
          Bh[qb] = pair8(Ph[qb][2 * kp], Ph[qb][2 * kp + 1]);
          if constexpr (kHiLo) Bl[qb] = pair8(Pl[qb][2 * kp], Pl[qb][2 * kp + 1]);
        }
#pragma unroll
        for (int cb = 0; cb < DVB; ++cb) {
          const bf16_t* vrow = Vt + (cb * 16 + c16) * kVtStride + kp * 32 + 4 * g4;
          const bf16x8_t A = pair8(*reinterpret_cast<const i16x4*>(vrow), *reinterpret_cast<const i16x4*>(vrow + 16));
#pragma unroll
          for (int qb = 0; qb < 2; ++qb) {
            O[qb][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A, Bh[qb], O[qb][cb], 0, 0, 0);
            if constexpr (kHiLo) O[qb][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A, Bl[qb], O[qb][cb], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    float l = lsum[qb];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!okrow[qb]) continue;
    const int r = 32 * w + 16 * qb + c16;
    if (a.sink && !a.wfn) l += fast_exp2(a.sink[qh] * kLog2e - mx[qb]);  // mx in log2 units, finite: a row sees itself
    float inv = a.wfn ? 1.f : 1.f / l;
    if (a.gate) inv /= 1.f + __expf(-bf16_to_f32(a.gate[(int64_t)(row0 + r) * a.gate_stride + head]));
    OutT* o = (OutT*)a.out + ((int64_t)(row0 + r) * a.n_qh + qh) * dv + 4 * g4;
#pragma unroll
    for (int cb = 0; cb < DVB; ++cb) store4<OutT>(o + cb * 16, O[qb][cb] * inv);
  }
}


// ---------------------------------------------------------------------------
// Decode rows: one wave per (row, K head, chunk of the heads that share it,
// key part).  The 16 B-operand columns are query heads of one group instead of
// 16 consecutive tokens, so the K/V bytes of a group are read once for all its
// heads; everything else is the tile kernel's arithmetic.  The wave's partial
// (max, sum, acc) go to the workspace that merge_parts (row_attention.hip)
// joins: ws [rows, n_qh, parts, 2 + dv].
struct GroupArgs {
  const bf16_t* q;
  int64_t q_stride;
  const bf16_t* kc;
  const bf16_t* vc;
  float* ws;
  const int64_t* pos;
  const int* seq;  // null: row i is sequence i
  const int* bt;
  int bt_stride, bs;
  int n_qh, maps, group, chunks;
  int Wk, Wv;
  float scale;
  int mask, size, parts;
  float softcap;
  const float* r1;
  const float* r2;
  int wfn;
  const float* hbias;
  int keep;  // window mask: the first `keep` keys of a sequence stay visible (0: none)
};

template <int DB, int DVB, int QB>
__global__ void __launch_bounds__(64) group_decode_kernel(GroupArgs a) {
  constexpr int d = DB * 16, dv = DVB * 16, ks_stride = d + 8;
  extern __shared__ __attribute__((aligned(16))) bf16_t smem[];
  bf16_t* Ks = smem;
  bf16_t* Vt = smem + kKeys * ks_stride;
  const int lane = threadIdx.x, c16 = lane & 15, g4 = lane >> 4;
  const int gm = blockIdx.x / a.chunks, chunk = blockIdx.x - gm * a.chunks;
  const int g = gm / a.maps, m = gm - g * a.maps;
  const int row = blockIdx.y, part = blockIdx.z;
  const int p = (int)a.pos[row];
  const int* bt = a.bt + (int64_t)(a.seq ? a.seq[row] : row) * a.bt_stride;
  const bf16_t* kc = a.kc + (int64_t)gm * d;
  const bf16_t* vc = a.vc + (int64_t)g * dv;
  const int lo = first_visible(p, a.mask, a.size);
  // the visible keys in one numbering: the kept first nf keys, then lo .. p (position u + shift)
  const int nf = a.mask == 1 && a.keep > 0 ? (a.keep < lo ? a.keep : lo) : 0;
  const int shift = lo - nf;
  const int tiles = (nf + p - lo + kKeys) / kKeys;
  const int tpp = (tiles + a.parts - 1) / a.parts;
  const int t0 = part * tpp, t1 = t0 + tpp < tiles ? t0 + tpp : tiles;

  i16x4 qf[QB][DB];
  bool okh[QB];
  int qh[QB];
  float r1[QB], r2[QB], hb[QB];
  const float cap = a.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int hi_ = chunk * 16 * QB + 16 * qb + c16;
    okh[qb] = hi_ < a.group;
    qh[qb] = (g * a.group + (okh[qb] ? hi_ : 0)) * a.maps + m;
    r1[qb] = a.r1 ? a.r1[qh[qb]] : 0.f;
    r2[qb] = a.r1 ? a.r2[qh[qb]] : 0.f;
    hb[qb] = a.hbias ? a.hbias[qh[qb]] : 0.f;
    const bf16_t* q = a.q + (int64_t)row * a.q_stride + (int64_t)qh[qb] * d + 4 * g4;
#pragma unroll
    for (int ks = 0; ks < DB; ++ks)
      qf[qb][ks] = okh[qb] ? *reinterpret_cast<const i16x4*>(q + ks * 16) : i16x4{0, 0, 0, 0};
  }
  float mx[QB], lsum[QB];
  f32x4 O[QB][DVB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    mx[qb] = a.wfn ? 0.f : -INFINITY;  // sigmoid weights: every part reports max 0 and sum 1
    lsum[qb] = 0.f;
#pragma unroll
    for (int cb = 0; cb < DVB; ++cb) O[qb][cb] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // wide heads: a whole tile in flight would not fit the register file beside the
  // accumulators, so K and V are staged one after the other and nothing is prefetched
  constexpr bool kWide = DB + DVB > 16;
  constexpr int VS = kWide ? kVtStrideWide : kVtStride;
  TileStage<d, dv, 64, VS> stage;
  if (!kWide && t0 < t1) stage.fetch(kc, vc, bt, a.bs, a.Wk, a.Wv, t0 * kKeys, nf, shift, p, lane);
  for (int t = t0; t < t1; ++t) {
    const int ut = t * kKeys;
    if constexpr (kWide) {
      stage.template fetch<true, false>(kc, vc, bt, a.bs, a.Wk, a.Wv, ut, nf, shift, p, lane);
      stage.template commit<true, false>(Ks, Vt, lane);
      stage.template fetch<false, true>(kc, vc, bt, a.bs, a.Wk, a.Wv, ut, nf, shift, p, lane);
      stage.template commit<false, true>(Ks, Vt, lane);
    } else {
      stage.commit(Ks, Vt, lane);
    }
    __syncthreads();
    if (!kWide && t + 1 < t1) stage.fetch(kc, vc, bt, a.bs, a.Wk, a.Wv, ut + kKeys, nf, shift, p, lane);
    f32x4 S[QB][4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) S[qb][kb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DB; ++ks) {
        const i16x4 A = *reinterpret_cast<const i16x4*>(Ks + (kb * 16 + c16) * ks_stride + ks * 16 + 4 * g4);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
          S[qb][kb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(A, qf[qb][ks], S[qb][kb], 0, 0, 0);
      }
    }
    i16x4 Ph[QB][4], Pl[QB][4];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mloc = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int ku = ut + kb * 16 + 4 * g4 + i, kj = ku < nf ? ku : ku + shift;
          float s = S[qb][kb][i] * a.scale;
          if (cap > 0.f) s = cap * (1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __expf(2.f * s * inv_cap)));
          if (a.r1) s -= r1[qb] * __logf(1.f + r2[qb] * (float)(p - kj > 0 ? p - kj : 0));
          s = kj <= p ? s + hb[qb] : -INFINITY;
          S[qb][kb][i] = s;
          mloc = fmaxf(mloc, s);
        }
      mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
      const float mn = a.wfn ? 0.f : fmaxf(mx[qb], mloc);  // finite: every visited tile holds a visible key
      const float alpha = __expf(mx[qb] - mn);              // sigmoid weights: 1
      mx[qb] = mn;
      float add = 0.f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        float pw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // sigmoid(s); an invisible key (s = -inf) weighs 1 / (1 + inf) = 0
          pw[i] = a.wfn ? __builtin_amdgcn_rcpf(1.f + __expf(-S[qb][kb][i])) : __expf(S[qb][kb][i] - mn);
          add += pw[i];
        }
        const uint32_t h01 = pack_bf16x2(pw[0], pw[1]), h23 = pack_bf16x2(pw[2], pw[3]);
        const uint32_t l01 = pack_bf16x2(pw[0] - bf16lo(h01), pw[1] - bf16hi(h01));
        const uint32_t l23 = pack_bf16x2(pw[2] - bf16lo(h23), pw[3] - bf16hi(h23));
        Ph[qb][kb] = __builtin_bit_cast(i16x4, uint2{h01, h23});
        Pl[qb][kb] = __builtin_bit_cast(i16x4, uint2{l01, l23});
      }
      lsum[qb] = lsum[qb] * alpha + add;
#pragma unroll
      for (int cb = 0; cb < DVB; ++cb) O[qb][cb] *= alpha;
    }
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int cb = 0; cb < DVB; ++cb) {
        const i16x4 A = *reinterpret_cast<const i16x4*>(Vt + (cb * 16 + c16) * VS + kb * 16 + 4 * g4);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
          O[qb][cb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(A, Ph[qb][kb], O[qb][cb], 0, 0, 0);
          O[qb][cb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(A, Pl[qb][kb], O[qb][cb], 0, 0, 0);
        }
      }
    __syncthreads();
  }
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    float l = lsum[qb];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!okh[qb]) continue;
    float* w = a.ws + (((int64_t)row * a.n_qh + qh[qb]) * a.parts + part) * (2 + dv);
    if (g4 == 0) {
      w[0] = mx[qb];
      w[1] = a.wfn ? 1.f : l;
    }
#pragma unroll
    for (int cb = 0; cb < DVB; ++cb)
#pragma unroll
      for (int i = 0; i < 4; ++i) w[2 + cb * 16 + 4 * g4 + i] = O[qb][cb][i];
  }
}

template <int DB, int DVB>
int launch_group(const GroupArgs& a0, int rows, hipStream_t st) {
  const size_t lds = (size_t)(kKeys * (DB * 16 + 8) + DVB * 16 * (DB + DVB > 16 ? kVtStrideWide : kVtStride)) * sizeof(bf16_t);
  GroupArgs a = a0;
  const bool two = a.group > 16 && DB + DVB <= 16;  // two head blocks per wave only where the registers hold them
  a.chunks = two ? (a.group + 31) / 32 : (a.group + 15) / 16;
  auto k1 = group_decode_kernel<DB, DVB, 1>;
  auto k2 = group_decode_kernel<DB, DVB, 2>;
  if (lds > 48 * 1024) {
    static bool raised = false;
    if (!raised) {
      if (hipFuncSetAttribute((const void*)k1, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess ||
          hipFuncSetAttribute((const void*)k2, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return 7;
      raised = true;
    }
  }
  const int n_gm = a.n_qh / a.group;  // K heads (kv heads x maps)
  const dim3 grid(n_gm * a.chunks, rows, a.parts);
  if (two) hipLaunchKernelGGL(k2, grid, dim3(64), lds, st, a);
  else hipLaunchKernelGGL(k1, grid, dim3(64), lds, st, a);
  DX_CHECK_LAUNCH();
  return 0;
}

template <int DB, int DVB, typename OutT>
int launch_tiles(const TileArgs& a, int n_tiles, hipStream_t st) {
  const size_t lds = (size_t)(kKeys * (DB * 16 + 8) + DVB * 16 * kVtStride) * sizeof(bf16_t);
  auto kern = tile_attention_kernel<DB, DVB, OutT>;
  if (lds > 48 * 1024) {
    static bool raised = false;  // per instantiation
    if (!raised) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return 7;
      raised = true;
    }
  }
  for (int t0 = 0; t0 < n_tiles; t0 += 65535) {
    TileArgs b = a;
    b.tiles = a.tiles + 2 * t0;
    const int nt = n_tiles - t0 < 65535 ? n_tiles - t0 : 65535;
    hipLaunchKernelGGL(kern, dim3(a.n_qh, nt), dim3(256), lds, st, b);
  }
  DX_CHECK_LAUNCH();
  return 0;
}

}  // namespace

#define TILE_CASE(DB_, DVB_)                                                               \
  if (d == DB_ * 16 && dv == DVB_ * 16)                                                    \
    return out_f32 ? launch_tiles<DB_, DVB_, float>(a, n_tiles, st) : launch_tiles<DB_, DVB_, bf16_t>(a, n_tiles, st);

extern "C" {

// 1 when tile_attention has an instance for the head widths
int dxm_tile_attention_ok(int d, int dv) {
  const int pairs[][2] = {{2, 2}, {2, 4}, {3, 3}, {3, 6}, {4, 4}, {4, 8}, {8, 8}, {8, 16}, {16, 12}, {16, 16}};
  for (auto& p : pairs)
    if (d == p[0] * 16 && dv == p[1] * 16) return 1;
  return 0;
}

int dxm_tile_attention(void* out, const void* q, int64_t q_stride, const void* kc, const void* vc, const int64_t* pos,
                       const int* seq, const int* bt, int bt_stride, int bs, const int* tiles, int n_tiles, int n_qh,
                       int maps, int group, int d, int dv, int Wk, int Wv, float scale, int mask, int size,
                       float softcap, const float* r1, const float* r2, int wfn, const float* hbias, const void* gate,
                       int64_t gate_stride, int keep, const float* sink, int out_f32, hipStream_t st) {
  if (n_tiles <= 0) return 0;
  if (softcap < 0.f || (r1 && !r2) || wfn < 0 || wfn > 1 || keep < 0 || (keep && mask != 1)) return 6;
  if (n_qh < 1 || maps < 1 || group < 1 || n_qh % maps || (n_qh / maps) % group || n_qh > 65535) return 1;
  if (mask < 0 || mask > 2 || (mask && size < 1) || !(scale > 0.f)) return 3;
  if (!seq || !tiles || Wk % 8 || Wv % 8 || q_stride % 8) return 4;
  TileArgs a{(const bf16_t*)q, q_stride, (const bf16_t*)kc, (const bf16_t*)vc, out, pos, seq, bt, bt_stride, bs,
             tiles, n_qh, maps, group, Wk, Wv, scale, mask, size, softcap, r1, r2, wfn, hbias, (const bf16_t*)gate,
             gate_stride, keep, sink};
  TILE_CASE(2, 2)
  TILE_CASE(2, 4)
  TILE_CASE(3, 3)
  TILE_CASE(3, 6)
  TILE_CASE(4, 4)
  TILE_CASE(4, 8)
  TILE_CASE(8, 8)
  TILE_CASE(8, 16)
  TILE_CASE(16, 12)
  TILE_CASE(16, 16)
  return 2;
}

#define GROUP_CASE(DB_, DVB_) \
  if (d == DB_ * 16 && dv == DVB_ * 16) return launch_group<DB_, DVB_>(a, rows, st);

// Decode rows (one token per row) on the matrix cores: partials into ws
// [rows, n_qh, parts, 2 + dv]; dxm_merge_parts joins them.
int dxm_group_decode(float* ws, const void* q, int64_t q_stride, const void* kc, const void* vc, const int64_t* pos,
                     const int* seq, const int* bt, int bt_stride, int bs, int rows, int n_qh, int maps, int group,
                     int d, int dv, int Wk, int Wv, float scale, int mask, int size, float softcap, const float* r1,
                     const float* r2, int wfn, const float* hbias, int keep, int parts, hipStream_t st) {
  if (rows <= 0) return 0;
  if (softcap < 0.f || (r1 && !r2) || wfn < 0 || wfn > 1 || keep < 0 || (keep && mask != 1)) return 6;
  if (n_qh < 1 || maps < 1 || group < 1 || n_qh % maps || (n_qh / maps) % group || rows > 65535) return 1;
  if (mask < 0 || mask > 2 || (mask && size < 1) || parts < 1 || parts > 65535) return 3;
  if (!ws || Wk % 8 || Wv % 8 || q_stride % 4) return 4;
  GroupArgs a{(const bf16_t*)q, q_stride, (const bf16_t*)kc, (const bf16_t*)vc, ws, pos, seq, bt, bt_stride, bs,
              n_qh, maps, group, 1, Wk, Wv, scale, mask, size, parts, softcap, r1, r2, wfn, hbias, keep};
  GROUP_CASE(2, 2)
  GROUP_CASE(2, 4)
  GROUP_CASE(3, 3)
  GROUP_CASE(3, 6)
  GROUP_CASE(4, 4)
  GROUP_CASE(4, 8)
  GROUP_CASE(8, 8)
  GROUP_CASE(8, 16)
  GROUP_CASE(16, 12)
  GROUP_CASE(16, 16)
  return 2;
}

}  // extern "C"
