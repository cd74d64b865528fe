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
//   a normaliser vector n_t = a_t n_{t-1} + b_t k_t rides along as one more state column (a
//   value that is always 1), q is scaled by d^(-1/2), and
//     o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//   is RMS-normed per head, times norm_w [H*dv], times sigmoid(gate_t), times out_scale -> S.
//
// Projection row of a token (fp32): [H*d q | H*d k | H*dv v | H*dv gate | H zi | H zf] (FORM 0
// reads q, k, v only). State: [slots, H, d, dve] with dve = dv (+ 1 for FORM 1); mstate
// [slots, H]. A step's tokens of one sequence are consecutive rows [cu[s], cu[s+1]);
// positions[cu[s]] == 0 starts from a zero state whatever the slot held; sequences with slot
// < 0 (padding rows of a captured decode step) get zeros.
//
// One workgroup per (head, sequence), thread c owns column c of the state. d in {16, 32, 64,
// 128}: the column lives in registers, its rows dealt to P thread groups (decode steps stream
// the state through them: one read, one write per element); any other d keeps the state in LDS.
// Tokens are taken in chunks of TC: activations and gates of the chunk in parallel (the gate
// scan by one thread), the walk without barriers, the chunk's read-outs finished one wave per
// token.
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

constexpr int TC = 16;

struct ScalarRecArgs {
  const float* proj; int ldp;
  const float* decays;            // [H] (FORM 0)
  const float* if_b; float cap;   // [2H] input | forget gate biases (FORM 1)
  const void* norm_w; float eps;  // [H*dv] (FORM 1)
  float* state; float* mstate;
  const int* slots; const int* cu; const int* positions;
  void* out; int ldo; float out_scale;
  int H, d, dv;
};

template <typename S, int D, int P, int FORM>
__global__ void __launch_bounds__(1024) scalar_recurrence_kernel(ScalarRecArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int H = a.H, d = a.d, dv = a.dv;
  const int dve = dv + (FORM == 1 ? 1 : 0);
  float* St = sm;                              // [d][dve] (D == 0 only)
  float* qv = St + (D ? 0 : d * dve);          // [TC][d]
  float* kv = qv + TC * d;                     // [TC][d]
  float* ov = kv + TC * d;                     // [P][TC][dve] (partial) read-outs
  float* vv = ov + P * TC * dve;               // [TC][dve] values (FORM 1: the last one is 1)
  float* ab = vv + TC * dve;                   // [TC][2] decay, input weight
  float* em = ab + 2 * TC;                     // [TC] exp(-m_t)
  constexpr int R = D ? D / P : 1;
  const int h = blockIdx.x, s = blockIdx.y;
  const int slot = a.slots[s];
  const int t0 = a.cu[s], t1 = a.cu[s + 1];
  const int dvp = blockDim.x / P;
  const int c = threadIdx.x % dvp, part = threadIdx.x / dvp;
  if (slot < 0) {
    for (int t = t0; t < t1; ++t)
      if (c < dv && part == 0) {
        if (FORM == 0) ((float*)a.out)[(long)t * a.ldo + h * dv + c] = 0.f;
        else stf((S*)a.out + (long)t * a.ldo + h * dv + c, 0.f);
      }
    return;
  }
  if (t1 <= t0) return;
  float* sp = a.state + ((long)slot * H + h) * d * dve;
  const bool fresh = a.positions[t0] == 0;
  float reg[R];
  if (D) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      reg[i] = (fresh || c >= dve) ? 0.f : sp[(long)(part * R + i) * dve + c];
  } else {
    for (int i = threadIdx.x; i < d * dve; i += blockDim.x) St[i] = fresh ? 0.f : sp[i];
  }
  float m_run = 0.f;                           // thread 0 carries the running maximum
  if (FORM == 1 && threadIdx.x == 0 && !fresh) m_run = a.mstate[(long)slot * H + h];
  const float qscale = FORM == 1 ? 1.f / sqrtf((float)d) : 1.f;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int voff = 2 * H * d + h * dv, goff = 2 * H * d + H * dv + h * dv;
  const int ioff = 2 * H * d + 2 * H * dv + h, foff = ioff + H;
  for (int tc = t0; tc < t1; tc += TC) {
    const int n = min(TC, t1 - tc);
    __syncthreads();                           // the previous chunk is done with ov / vv / ab
    for (int i = threadIdx.x; i < n * dve; i += blockDim.x) {
      const int tt = i / dve, cc = i % dve;
      float v = 1.f;
      if (cc < dv) {
        v = a.proj[(long)(tc + tt) * a.ldp + voff + cc];
        if (FORM == 0) v = silu32(v);
      }
      vv[i] = v;
    }
    for (int i = threadIdx.x; i < n * d; i += blockDim.x) {
      const float* row = a.proj + (long)(tc + i / d) * a.ldp + h * d + i % d;
      const float q = row[0], k = row[H * d];
      qv[i] = FORM == 0 ? silu32(q) : q * qscale;
      kv[i] = FORM == 0 ? silu32(k) : k;
    }
    if (FORM == 0) {
      if (threadIdx.x < n) { ab[2 * threadIdx.x] = a.decays[h]; ab[2 * threadIdx.x + 1] = 1.f; }
    } else if (threadIdx.x == 0) {
      const float bi = a.if_b[h], bf = a.if_b[H + h];
      for (int tt = 0; tt < n; ++tt) {
        const float* row = a.proj + (long)(tc + tt) * a.ldp;
        const float ig = a.cap * tanhf((row[ioff] + bi) / a.cap);
        const float fg = logsigmoid32(a.cap * tanhf((row[foff] + bf) / a.cap));
        const float m1 = fmaxf(fg + m_run, ig);
        ab[2 * tt] = expf(fg + m_run - m1);
        ab[2 * tt + 1] = expf(ig - m1);
        em[tt] = expf(-m1);
        m_run = m1;
      }
    }
    __syncthreads();
    if (c < dve) {
#pragma unroll 1
      for (int tt = 0; tt < n; ++tt) {
        const float at = ab[2 * tt];
        const float bv = ab[2 * tt + 1] * vv[tt * dve + c];
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
            const float sv = at * St[i * dve + c] + k[i] * bv;
            St[i * dve + c] = sv;
            o += sv * q[i];
          }
        }
        ov[(part * TC + tt) * dve + c] = o;
      }
    }
    __syncthreads();
    for (int tt = wid; tt < n; tt += nw) {
      const long t = tc + tt;
      if (FORM == 0) {
        for (int k = lane; k < dv; k += 64) {
          float o = ov[tt * dve + k];
#pragma unroll
          for (int pp = 1; pp < P; ++pp) o += ov[(pp * TC + tt) * dve + k];
          ((float*)a.out)[t * a.ldo + h * dv + k] = o;
        }
      } else {
        float nq = ov[tt * dve + dv];
#pragma unroll
        for (int pp = 1; pp < P; ++pp) nq += ov[(pp * TC + tt) * dve + dv];
        const float den = fmaxf(fabsf(nq), em[tt]) + 1e-6f;
        float ss = 0.f;
        for (int k = lane; k < dv; k += 64) {
          float o = ov[tt * dve + k];
#pragma unroll
          for (int pp = 1; pp < P; ++pp) o += ov[(pp * TC + tt) * dve + k];
          o = o / den;
          ov[tt * dve + k] = o;
          ss += o * o;
        }
        ss = wave_sum(ss);
        const float rs = 1.f / sqrtf(ss / (float)dv + a.eps);
        for (int k = lane; k < dv; k += 64) {
          const float g = a.proj[t * a.ldp + goff + k];
          const float val = ov[tt * dve + k] * rs * ldf((const S*)a.norm_w + h * dv + k) *
                            (1.f / (1.f + expf(-g))) * a.out_scale;
          stf((S*)a.out + t * a.ldo + h * dv + k, val);
        }
      }
    }
  }
  if (FORM == 1 && threadIdx.x == 0) a.mstate[(long)slot * H + h] = m_run;
  if (D) {
    if (c < dve) {
#pragma unroll
      for (int i = 0; i < R; ++i) sp[(long)(part * R + i) * dve + c] = reg[i];
    }
    return;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < d * dve; i += blockDim.x) sp[i] = St[i];
}

template <typename S, int FORM>
int launch_scalar_recurrence(const ScalarRecArgs& a, int num_seqs, hipStream_t st) {
  const int d = a.d, dve = a.dv + (FORM == 1 ? 1 : 0);
  const int threads = ((dve + 63) / 64) * 64;
  if (threads > 1024) return (int)hipErrorInvalidValue;
  int D = (d == 16 || d == 32 || d == 64 || d == 128) ? d : 0;
  const int P = D >= 64 ? 4 : (D == 32 ? 2 : 1);
  if (D && threads * P > 1024) D = 0;
  const int nthreads = D ? threads * P : threads;
  const size_t sh = ((size_t)(D ? 0 : d * dve) + 2 * (size_t)TC * d +
                     (size_t)((D ? P : 1) + 1) * TC * dve + 3 * TC) * 4;
  if (sh > 160 * 1024) return (int)hipErrorInvalidValue;
  dim3 grid(a.H, num_seqs);
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
    case 128: SR_LAUNCH(128, 4); break;
    default: SR_LAUNCH(0, 1); break;
  }
#undef SR_LAUNCH
  DLI_RETURN_LAUNCH();
}

}  // namespace

// form 0: fixed-decay linear attention (out fp32 [T, H*dv], dt ignored); form 1: matrix memory
// with exponential gating (out in the storage type dt, norm_w likewise).
extern "C" int dli_scalar_recurrence(const float* proj, int ldp, int form, const float* decays,
                                     const float* if_b, float cap, const void* norm_w, float eps,
                                     float* state, float* mstate, const int* slots, const int* cu,
                                     const int* positions, void* out, int ldo, float out_scale,
                                     int num_seqs, int max_seqlen, int H, int d, int dv, int dt,
                                     hipStream_t st) {
  if (num_seqs <= 0 || max_seqlen <= 0) return 0;
  if (H < 1 || d < 1 || dv < 1 || state == nullptr || out == nullptr)
    return (int)hipErrorInvalidValue;
  ScalarRecArgs a{proj, ldp, decays, if_b, cap, norm_w, eps, state, mstate, slots, cu, positions,
                  out, ldo, out_scale, H, d, dv};
  if (form == 0) {
    if (decays == nullptr) return (int)hipErrorInvalidValue;
    return launch_scalar_recurrence<float, 0>(a, num_seqs, st);
  }
  if (form != 1 || if_b == nullptr || norm_w == nullptr || mstate == nullptr || !(cap > 0.f))
    return (int)hipErrorInvalidValue;
  if (dt == 0) return launch_scalar_recurrence<u16, 1>(a, num_seqs, st);
  if (dt == 1) return launch_scalar_recurrence<float, 1>(a, num_seqs, st);
  return (int)hipErrorInvalidValue;
}
