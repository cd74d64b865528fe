// Linear recurrences whose decay is one number per head and token, with per-sequence fp32
// state slots:
//     S_t = a_t S_{t-1} + b_t k_t v_t^T,      o_t = S_t^T q_t          S [d, dv] per head
//
// FORM 0, fixed-decay linear attention: a_t = decay[h], b_t = 1; q, k, v pass through SiLU;
//   the raw read-outs leave in fp32 (the caller norms all heads of a token together).
// FORM 1, matrix memory with exponential gating: with the soft-capped gate pre-activations
//     i_t = cap tanh((zi_t + bi) / cap),   f_t = logsigmoid(cap tanh((zf_t + bf) / cap))
//   and a running maximum m (0 at a sequence's start):
//     m_t = max(f_t + m_{t-1}, i_t),   a_t = exp(f_t + m_{t-1} - m_t),   b_t = exp(i_t - m_t)
//   a normaliser vector n_t = a_t n_{t-1} + b_t k_t rides along, q is scaled by d^(-1/2), and
//     o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//   is RMS-normed per head, times norm_w [H*dv], times sigmoid(gate_t), times out_scale -> S.
//   n_t . q_t needs no state column of its own: inside a chunk of tokens
//     n_t . q_t = A_t (n_0 . q_t) + sum_{j <= t} b_j (prod_{j < i <= t} a_i) (k_j . q_t),
//   A_t = prod_{i <= t} a_i, so the chunk's key-query products and the carried vector n_0 (LDS,
//   updated once a chunk) give every token's normaliser in parallel, beside the walk.
//
// Projection row of a token (fp32): [H*d q | H*d k | H*dv v | H*dv gate | H zi | H zf] (FORM 0
// reads q, k, v only). State: [slots, H, d, dv]; FORM 1 also nstate [slots, H, d + 1] = n, then
// m. A step's tokens of one sequence are consecutive rows [cu[s], cu[s+1]);
// positions[cu[s]] == 0 starts from a zero state whatever the slot held; sequences with slot
// < 0 (padding rows of a captured decode step) get zeros.
//
// One workgroup per (head, sequence, block of cw state columns), thread c owns one column. d
// in {16, 32, 64, 128}: the column lives in registers, its rows dealt to P thread groups
// (decode steps stream the state through them: one read, one write per element); any other d
// keeps the state in LDS. Tokens are taken in chunks of TC: activations and gates of the
// chunk in parallel (the running maximum by one wave), the walk without barriers, the
// chunk's read-outs finished one wave per token. With several column blocks a head's RMS norm
// cannot happen here: FORM 1 then leaves o_t in fp32 (`raw`) for a norm kernel.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float silu32(float g) { return g / (1.f + expf(-g)); }
// log(sigmoid(x)), stable on both sides
__device__ __forceinline__ float logsigmoid32(float x) {
  return x > 0.f ? -log1pf(expf(-x)) : x - log1pf(expf(x));
}

// tokens per chunk (32 was measured: the walk gains little, the matrix memory's per-chunk
// products and scans, which grow with the square of the chunk, lose more)
constexpr int TC = 16;

struct ScalarRecArgs {
  const float* proj; int ldp;
  const float* decays;            // [H] (FORM 0)
  const float* if_b; float cap;   // [2H] input | forget gate biases (FORM 1)
  const void* norm_w; float eps;  // [H*dv] (FORM 1)
  float* state; float* nstate;
  const int* slots; const int* cu; const int* positions;
  void* out; int ldo; float out_scale;
  float* raw;                     // FORM 1, several column blocks: o_t in fp32 [T, H*dv]
  int H, d, dv, cw;               // cw: state columns per workgroup
};

template <typename S, int D, int P, int FORM>
__global__ void __launch_bounds__(1024) scalar_recurrence_kernel(ScalarRecArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int H = a.H, d = a.d, dv = a.dv;
  const int dvp = blockDim.x / P;              // column threads of a row group
  const int c0 = blockIdx.z * a.cw, ncol = min(a.cw, dv - c0);
  float* St = sm;                              // [d][dvp] (D == 0 only)
  float* qv = St + (D ? 0 : d * dvp);          // [TC][d]
  float* kv = qv + TC * d;                     // [TC][d]
  float* ov = kv + TC * d;                     // [P][TC][dvp] (partial) read-outs
  float* vv = ov + P * TC * dvp;               // [TC][dvp] values
  float* ab = vv + TC * dvp;                   // [TC][2] decay, input weight
  float* em = ab + 2 * TC;                     // [TC] exp(-m_t)
  float* gi = em + TC;                         // [TC] log input gate
  float* gf = gi + TC;                         // [TC] log forget gate
  float* den = gf + TC;                        // [TC] the read-out's denominator
  float* n0q = den + TC;                       // [TC] n_0 . q_t
  float* kq = n0q + TC;                        // [TC][TC] k_j . q_t
  float* nvec = kq + TC * TC;                  // [d] the normaliser at the chunk's start
  constexpr int R = D ? D / P : 1;
  const int h = blockIdx.x, s = blockIdx.y;
  const int slot = a.slots[s];
  const int t0 = a.cu[s], t1 = a.cu[s + 1];
  const int c = threadIdx.x % dvp, part = threadIdx.x / dvp;
  const bool fused_norm = FORM == 1 && a.raw == nullptr;
  if (slot < 0) {
    for (int t = t0; t < t1; ++t)
      if (c < ncol && part == 0) {
        if (FORM == 0) ((float*)a.out)[(long)t * a.ldo + h * dv + c0 + c] = 0.f;
        else if (fused_norm) stf((S*)a.out + (long)t * a.ldo + h * dv + c0 + c, 0.f);
        else a.raw[(long)t * H * dv + h * dv + c0 + c] = 0.f;
      }
    return;
  }
  if (t1 <= t0) return;
  float* sp = a.state + ((long)slot * H + h) * d * dv + c0;
  float* np = FORM == 1 ? a.nstate + ((long)slot * H + h) * (d + 1) : nullptr;
  const bool fresh = a.positions[t0] == 0;
  float reg[R];
  if (D) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      reg[i] = (fresh || c >= ncol) ? 0.f : sp[(long)(part * R + i) * dv + c];
  } else {
    for (int i = threadIdx.x; i < d * dvp; i += blockDim.x)
      St[i] = (fresh || i % dvp >= ncol) ? 0.f : sp[(long)(i / dvp) * dv + i % dvp];
  }
  float m_run = 0.f;                           // the running maximum (wave 0 carries it)
  if (FORM == 1) {
    if (!fresh) m_run = np[d];
    for (int i = threadIdx.x; i < d; i += blockDim.x) nvec[i] = fresh ? 0.f : np[i];
  }
  const float qscale = FORM == 1 ? 1.f / sqrtf((float)d) : 1.f;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int voff = 2 * H * d + h * dv + c0, goff = 2 * H * d + H * dv + h * dv + c0;
  const int ioff = 2 * H * d + 2 * H * dv + h, foff = ioff + H;
  for (int tc = t0; tc < t1; tc += TC) {
    const int n = min(TC, t1 - tc);
    __syncthreads();                           // the previous chunk is done with the LDS rows
    // (thread = (row group `part`, column c): token part + u P, column c — no divisions; with
    // the rows in registers d is the constant D, a power of two)
    for (int tt = part; tt < n; tt += P) {
      float v = 0.f;
      if (c < ncol) {
        v = a.proj[(long)(tc + tt) * a.ldp + voff + c];
        if (FORM == 0) v = silu32(v);
      }
      vv[tt * dvp + c] = v;
    }
    const int dd = D ? D : d;
    for (int i = threadIdx.x; i < n * dd; i += blockDim.x) {
      const float* row = a.proj + (long)(tc + i / dd) * a.ldp + h * dd + i % dd;
      const float q = row[0], k = row[H * dd];
      qv[i] = FORM == 0 ? silu32(q) : q * qscale;
      kv[i] = FORM == 0 ? silu32(k) : k;
    }
    if (FORM == 0) {
      if (threadIdx.x < n) { ab[2 * threadIdx.x] = a.decays[h]; ab[2 * threadIdx.x + 1] = 1.f; }
    } else {
      if (threadIdx.x < n) {                   // the gates' logarithms, a token a thread
        const float* row = a.proj + (long)(tc + threadIdx.x) * a.ldp;
        gi[threadIdx.x] = a.cap * tanhf((row[ioff] + a.if_b[h]) / a.cap);
        gf[threadIdx.x] = logsigmoid32(a.cap * tanhf((row[foff] + a.if_b[H + h]) / a.cap));
      }
      __syncthreads();
      if (wid == 0) {                          // the maximum's scan: n short steps, every lane alike
        for (int tt = 0; tt < n; ++tt) {
          const float fg = gf[tt], ig = gi[tt];
          const float m1 = fmaxf(fg + m_run, ig);
          if (lane == tt) {
            ab[2 * tt] = expf(fg + m_run - m1);
            ab[2 * tt + 1] = expf(ig - m1);
            em[tt] = expf(-m1);
          }
          m_run = m1;
        }
      }
      // k_j . q_t for j <= t, and n_0 . q_t
      for (int idx = threadIdx.x; idx < TC * TC + TC; idx += blockDim.x) {
        const int tt = idx < TC * TC ? idx / TC : idx - TC * TC;
        const int j = idx < TC * TC ? idx % TC : -1;
        if (tt >= n || j > tt) continue;
        const float* q = qv + tt * dd;
        const float* k = j < 0 ? nvec : kv + j * dd;
        // rows are d floats apart (a multiple of the bank count for the usual d): every
        // thread starts its walk at another element, so a wave's reads fall into distinct banks
        float acc = 0.f;
        int ii = idx % dd;
        for (int i = 0; i < dd; ++i) {
          acc += k[ii] * q[ii];
          ii = ii + 1 == dd ? 0 : ii + 1;
        }
        if (j < 0) n0q[tt] = acc; else kq[idx] = acc;
      }
    }
    __syncthreads();
    if (FORM == 1) {
      if (threadIdx.x < n) {                   // this token's normaliser and denominator
        const int tt = threadIdx.x;
        float acc = 0.f, prod = 1.f;
        for (int j = tt; j >= 0; --j) {
          acc += ab[2 * j + 1] * prod * kq[tt * TC + j];
          prod *= ab[2 * j];
        }
        den[tt] = fmaxf(fabsf(prod * n0q[tt] + acc), em[tt]) + 1e-6f;
      }
      for (int i = threadIdx.x; i < d; i += blockDim.x) {   // n at the chunk's end
        float acc = 0.f, prod = 1.f;
        for (int j = n - 1; j >= 0; --j) {
          acc += ab[2 * j + 1] * prod * kv[j * d + i];
          prod *= ab[2 * j];
        }
        nvec[i] = prod * nvec[i] + acc;
      }
    }
    if (c < ncol) {
#pragma unroll 1
      for (int tt = 0; tt < n; ++tt) {
        const float at = ab[2 * tt];
        const float bv = ab[2 * tt + 1] * vv[tt * dvp + c];
        const float* q = qv + tt * d;
        const float* k = kv + tt * d;
        float o = 0.f;
        if (D) {
#pragma unroll
          for (int i = 0; i < R; i += 4) {
            const f32x4 q4 = *reinterpret_cast<const f32x4*>(q + part * R + i);
            const f32x4 k4 = *reinterpret_cast<const f32x4*>(k + part * R + i);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              reg[i + u] = at * reg[i + u] + k4[u] * bv;
              o += reg[i + u] * q4[u];
            }
          }
        } else {
          for (int i = 0; i < d; ++i) {
            const float sv = at * St[i * dvp + c] + k[i] * bv;
            St[i * dvp + c] = sv;
            o += sv * q[i];
          }
        }
        ov[(part * TC + tt) * dvp + c] = o;
      }
    }
    __syncthreads();
    for (int tt = wid; tt < n; tt += nw) {
      const long t = tc + tt;
      if (FORM == 0) {
        for (int k = lane; k < ncol; k += 64) {
          float o = ov[tt * dvp + k];
#pragma unroll
          for (int pp = 1; pp < P; ++pp) o += ov[(pp * TC + tt) * dvp + k];
          ((float*)a.out)[t * a.ldo + h * dv + c0 + k] = o;
        }
      } else {
        const float inv = 1.f / den[tt];
        float ss = 0.f;
        for (int k = lane; k < ncol; k += 64) {
          float o = ov[tt * dvp + k];
#pragma unroll
          for (int pp = 1; pp < P; ++pp) o += ov[(pp * TC + tt) * dvp + k];
          o *= inv;
          if (fused_norm) { ov[tt * dvp + k] = o; ss += o * o; }
          else a.raw[t * H * dv + h * dv + c0 + k] = o;
        }
        if (!fused_norm) continue;
        ss = wave_sum(ss);
        const float rs = 1.f / sqrtf(ss / (float)dv + a.eps);
        for (int k = lane; k < ncol; k += 64) {
          const float g = a.proj[t * a.ldp + goff + k];
          const float val = ov[tt * dvp + k] * rs * ldf((const S*)a.norm_w + h * dv + k) *
                            (1.f / (1.f + expf(-g))) * a.out_scale;
          stf((S*)a.out + t * a.ldo + h * dv + k, val);
        }
      }
    }
  }
  if (FORM == 1 && blockIdx.z == 0) {          // every column block carries the same n and m
    if (threadIdx.x == 0) np[d] = m_run;
    for (int i = threadIdx.x; i < d; i += blockDim.x) np[i] = nvec[i];
  }
  if (D) {
    if (c < ncol) {
#pragma unroll
      for (int i = 0; i < R; ++i) sp[(long)(part * R + i) * dv + c] = reg[i];
    }
    return;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < d * dvp; i += blockDim.x)
    if (i % dvp < ncol) sp[(long)(i / dvp) * dv + i % dvp] = St[i];
}

template <typename S, int FORM>
int launch_scalar_recurrence(const ScalarRecArgs& a, int num_seqs, hipStream_t st) {
  const int d = a.d;
  const int cols = a.cw < a.dv ? a.cw : a.dv;
  const int threads = ((cols + 63) / 64) * 64;
  if (threads > 1024) return (int)hipErrorInvalidValue;
  int D = (d == 16 || d == 32 || d == 64 || d == 128) ? d : 0;
  int P = D >= 64 ? 4 : (D == 32 ? 2 : 1);
  if (D == 128 && threads * 8 <= 512) P = 8;   // narrow column blocks: more row groups
  if (D && threads * P > 1024) D = 0;
  const int nthreads = D ? threads * P : threads;
  const size_t sh = ((size_t)(D ? 0 : d * threads) + 2 * (size_t)TC * d +
                     (size_t)((D ? P : 1) + 1) * TC * threads + 7 * TC + TC * TC + d) * 4;
  if (sh > 160 * 1024) return (int)hipErrorInvalidValue;
  dim3 grid(a.H, num_seqs, (a.dv + cols - 1) / cols);
#define SR_LAUNCH(DD, PP)                                                                       \
  do {                                                                                          \
    if (sh > 48 * 1024) {                                                                       \
      hipError_t e = hipFuncSetAttribute((const void*)scalar_recurrence_kernel<S, DD, PP, FORM>, \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh);  \
      if (e != hipSuccess) return (int)e;                                                       \
    }                                                                                           \
    scalar_recurrence_kernel<S, DD, PP, FORM><<<grid, nthreads, sh, st>>>(a);                   \
  } while (0)
  switch (D) {
    case 16: SR_LAUNCH(16, 1); break;
    case 32: SR_LAUNCH(32, 2); break;
    case 64: SR_LAUNCH(64, 4); break;
    case 128: if (P == 8) SR_LAUNCH(128, 8); else SR_LAUNCH(128, 4); break;
    default: SR_LAUNCH(0, 1); break;
  }
#undef SR_LAUNCH
  DLI_RETURN_LAUNCH();
}

}  // namespace

// form 0: fixed-decay linear attention (out fp32 [T, H*dv], dt ignored); form 1: matrix memory
// with exponential gating (out in the storage type dt, norm_w likewise). cw > 0 deals the
// state's columns to workgroups in blocks of cw (a multiple of 64); form 1 then writes o_t
// (before the head norm) to raw [T, H*dv] in fp32 and leaves norm, gate and scale to the caller.
extern "C" int dli_scalar_recurrence(const float* proj, int ldp, int form, const float* decays,
                                     const float* if_b, float cap, const void* norm_w, float eps,
                                     float* state, float* nstate, const int* slots, const int* cu,
                                     const int* positions, void* out, int ldo, float out_scale,
                                     int num_seqs, int max_seqlen, int H, int d, int dv, int cw,
                                     float* raw, int dt, hipStream_t st) {
  if (num_seqs <= 0 || max_seqlen <= 0) return 0;
  if (H < 1 || d < 1 || dv < 1 || state == nullptr || cw < 0 || (cw > 0 && cw % 64))
    return (int)hipErrorInvalidValue;
  if (cw == 0 || cw >= dv) { cw = dv; raw = form == 1 ? nullptr : raw; }
  ScalarRecArgs a{proj, ldp, decays, if_b, cap, norm_w, eps, state, nstate, slots, cu, positions,
                  out, ldo, out_scale, raw, H, d, dv, cw};
  if (form == 0) {
    if (decays == nullptr || out == nullptr) return (int)hipErrorInvalidValue;
    return launch_scalar_recurrence<float, 0>(a, num_seqs, st);
  }
  if (form != 1 || if_b == nullptr || norm_w == nullptr || nstate == nullptr || !(cap > 0.f) ||
      (cw < dv) != (raw != nullptr) || (raw == nullptr && out == nullptr))
    return (int)hipErrorInvalidValue;
  if (dt == 0) return launch_scalar_recurrence<u16, 1>(a, num_seqs, st);
  if (dt == 1) return launch_scalar_recurrence<float, 1>(a, num_seqs, st);
  return (int)hipErrorInvalidValue;
}
