// Gated linear recurrence (HGRN2 form) with per-sequence fp32 state slots.
//
// Per head, with state S [d, dv] (fp32, one slot per live sequence and layer run):
//     f_t = lower + (1 - lower) * sigmoid(fz_t + f_bias)          forget gate per channel, fp32
//     S_t = diag(f_t) S_{t-1} + (1 - f_t) v_t^T                    (1 - f) is what gets written
//     o_t = S_t^T silu(qz_t)
//     out_t = o_t / sqrt(mean(o_t^2) + eps) * norm_w               RMS norm over dv, per head
// The projection row of a token is [H*d qz | H*d fz | H*dv v] in fp32. A step's tokens of one
// sequence are consecutive rows [cu[s], cu[s+1]); positions[cu[s]] == 0 marks a sequence's
// first portion, which starts from a zero state whatever the slot held before (slots are
// reused without clearing). Sequences with slot < 0 (padding rows of a captured decode step)
// are skipped.
//
// The same kernels run gated linear attention (GLA = true), whose keys are independent of the
// decay:
//     a_t = sigmoid(z_t + a_bias)^(1/tau) = exp(-softplus(-(z_t + a_bias)) / tau)      fp32
//     S_t = diag(a_t) S_{t-1} + k_t v_t^T,   o_t = S_t^T (q_t * qscale)
//     out_t = o_t / sqrt(mean(o_t^2) + eps) * norm_w * silu(gate_t)
// with the projection row [H*d q | H*d k | H*dv v | H*dv gate | ...] and the decay's
// pre-activation z [T, H*d] in a buffer of its own.
//
// Two kernels, one workgroup per (head, sequence), thread c owns column c of the state: decode
// steps stream the state through registers (read once, written once); portions keep it in
// LDS and walk their tokens in chunks (the walk is sequential in time by the recurrence's
// per-channel decay; the gates and the norm of a chunk are computed in parallel).
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// sigmoid(x)^(inv_tau) through the logarithm: exp(-softplus(-x) * inv_tau), stable on both sides
__device__ __forceinline__ float decay_pow(float x, float inv_tau) {
  const float sp = x > 0.f ? log1pf(expf(-x)) : -x + log1pf(expf(x));
  return expf(-sp * inv_tau);
}

__device__ __forceinline__ float silu32(float g) { return g / (1.f + expf(-g)); }

constexpr int TC = 16;   // tokens per chunk of the portion kernel

// Portions: the state of one (sequence, head) lives in LDS for the whole portion; tokens are
// taken in chunks of TC: (1) every thread helps turning the chunk's q / f pre-activations into
// silu(q) and the forget gate, (2) thread c walks the chunk's tokens over its state column
// without any barrier, (3) the chunk's read-outs are RMS-normed, one wave per token.
// D > 0: d == D and the state lives in registers: the block is P groups of dvp = round64(dv)
// threads, thread (c, part) owns rows [part * D/P, (part+1) * D/P) of column c (fully unrolled
// walk); the P partial read-outs of a token meet in LDS at the chunk's end.
// D == 0: any d, the state lives in LDS (P = 1).
template <typename S, int D, int P, bool GLA>
__global__ void __launch_bounds__(1024) hgrn2_kernel(const float* __restrict__ proj, int ldp, const S* __restrict__ f_bias,
                             const S* __restrict__ lower, const S* __restrict__ norm_w, float eps,
                             float* __restrict__ state, const int* __restrict__ slots,
                             const int* __restrict__ cu, const int* __restrict__ positions,
                             S* __restrict__ out, int ldo, int H, int d, int dv,
                             const float* __restrict__ zp, int ldz, float inv_tau, float qscale) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  float* St = sm;                 // [d][dv] (D == 0 only)
  float* qv = St + (D ? 0 : d * dv);   // [TC][d] silu(qz) (GLA: q * qscale)
  float* fv = qv + TC * d;        // [TC][d] forget gate (GLA: the decay)
  float* ov = fv + TC * d;        // [P][TC][dv] (partial) read-outs of the chunk
  float* vv = ov + P * TC * dv;   // [TC][dv] the chunk's values
  float* kv = vv + TC * dv;       // [TC][d] the chunk's keys (GLA only)
  constexpr int R = D ? D / P : 1;
  const int h = blockIdx.x, s = blockIdx.y;
  const int slot = slots[s];
  const int t0 = cu[s], t1 = cu[s + 1];
  const int dvp = blockDim.x / P;
  const int c = threadIdx.x % dvp, part = threadIdx.x / dvp;
  if (slot < 0) {                        // padding rows: defined (zero) output, no state
    for (int t = t0; t < t1; ++t)
      if (c < dv && part == 0) stf(out + (long)t * ldo + h * dv + c, 0.f);
    return;
  }
  if (t1 <= t0) return;
  float* sp = state + ((long)slot * H + h) * d * dv;
  const bool fresh = positions[t0] == 0;
  float reg[R];
  if (D) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      reg[i] = (fresh || c >= dv) ? 0.f : sp[(long)(part * R + i) * dv + c];
  } else {
    for (int i = threadIdx.x; i < d * dv; i += blockDim.x) St[i] = fresh ? 0.f : sp[i];
  }
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int tc = t0; tc < t1; tc += TC) {
    const int n = min(TC, t1 - tc);
    __syncthreads();                     // previous chunk's norm phase is done with ov
    for (int i = threadIdx.x; i < n * dv; i += blockDim.x)
      vv[i] = proj[(long)(tc + i / dv) * ldp + 2 * H * d + h * dv + i % dv];
    for (int i0 = threadIdx.x; i0 < n * d; i0 += 4 * blockDim.x) {
      float qz[4], fz[4];                // 8 loads in flight per thread
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = i0 + u * blockDim.x;
        qz[u] = fz[u] = 0.f;
        if (i < n * d) {
          const float* row = proj + (long)(tc + i / d) * ldp + h * d + i % d;
          qz[u] = row[0];
          fz[u] = row[H * d];                  // GLA: the key
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = i0 + u * blockDim.x;
        if (i < n * d) {
          const int k = i % d;
          if (GLA) {
            qv[i] = qz[u] * qscale;
            kv[i] = fz[u];
            fv[i] = decay_pow(zp[(long)(tc + i / d) * ldz + h * d + k] + ldf(f_bias + h * d + k),
                              inv_tau);
          } else {
            qv[i] = qz[u] / (1.f + expf(-qz[u]));
            const float lw = ldf(lower + h * d + k);
            fv[i] = lw + (1.f - lw) / (1.f + expf(-(fz[u] + ldf(f_bias + h * d + k))));
          }
        }
      }
    }
    __syncthreads();
    if (c < dv) {
#pragma unroll 1
      for (int tt = 0; tt < n; ++tt) {
        const float v = vv[tt * dv + c];
        const float* q = qv + tt * d;
        const float* f = fv + tt * d;
        const float* kk = kv + tt * d;
        float o = 0.f;
        if (D) {
#pragma unroll
          for (int i = 0; i < R; i += 4) {
            const f32x4 f4 = *reinterpret_cast<const f32x4*>(f + part * R + i);
            const f32x4 q4 = *reinterpret_cast<const f32x4*>(q + part * R + i);
            f32x4 k4;
            if (GLA) k4 = *reinterpret_cast<const f32x4*>(kk + part * R + i);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              reg[i + u] = f4[u] * reg[i + u] + (GLA ? k4[u] : 1.f - f4[u]) * v;
              o += reg[i + u] * q4[u];
            }
          }
        } else {
          for (int i = 0; i < d; ++i) {
            const float fi = f[i];
            const float sv = fi * St[i * dv + c] + (GLA ? kk[i] : 1.f - fi) * v;
            St[i * dv + c] = sv;
            o += sv * q[i];
          }
        }
        ov[(part * TC + tt) * dv + c] = o;
      }
    }
    __syncthreads();
    for (int tt = wid; tt < n; tt += nw) {
      float ss = 0.f;
      for (int k = lane; k < dv; k += 64) {
        float o = ov[tt * dv + k];
#pragma unroll
        for (int pp = 1; pp < P; ++pp) o += ov[(pp * TC + tt) * dv + k];
        ov[tt * dv + k] = o;
        ss += o * o;
      }
      ss = wave_sum(ss);
      const float rs = 1.f / sqrtf(ss / (float)dv + eps);
      for (int k = lane; k < dv; k += 64) {
        float val = ov[tt * dv + k] * rs * ldf(norm_w + k);
        if (GLA) val *= silu32(proj[(long)(tc + tt) * ldp + 2 * H * d + H * dv + h * dv + k]);
        stf(out + (long)(tc + tt) * ldo + h * dv + k, val);
      }
    }
  }
  if (D) {
    if (c < dv) {
#pragma unroll
      for (int i = 0; i < R; ++i) sp[(long)(part * R + i) * dv + c] = reg[i];
    }
    return;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < d * dv; i += blockDim.x) sp[i] = St[i];
}

// Decode steps (every sequence brings one token): the state streams through registers, one
// read and one write per element, no LDS copy. One workgroup per (head, sequence), thread c
// owns column c: consecutive threads touch consecutive addresses of every state row.
template <typename S, bool GLA>
__global__ void hgrn2_step_kernel(const float* __restrict__ proj, int ldp,
                                  const S* __restrict__ f_bias, const S* __restrict__ lower,
                                  const S* __restrict__ norm_w, float eps,
                                  float* __restrict__ state, const int* __restrict__ slots,
                                  const int* __restrict__ cu, const int* __restrict__ positions,
                                  S* __restrict__ out, int ldo, int H, int d, int dv,
                                  const float* __restrict__ zp, int ldz, float inv_tau,
                                  float qscale) {
  extern __shared__ float sm[];
  float* qv = sm;                 // [d]
  float* fv = qv + d;             // [d]
  float* red = fv + d;            // [16]
  float* kv = red + 16;           // [d] keys (GLA only)
  const int h = blockIdx.x, s = blockIdx.y;
  const int slot = slots[s];
  const int t = cu[s];
  const int c = threadIdx.x;
  if (cu[s + 1] <= t) return;
  if (slot < 0) {
    if (c < dv) stf(out + (long)t * ldo + h * dv + c, 0.f);
    return;
  }
  const float* row = proj + (long)t * ldp;
  for (int k = c; k < d; k += blockDim.x) {
    const float qz = row[h * d + k];
    if (GLA) {
      qv[k] = qz * qscale;
      kv[k] = row[H * d + h * d + k];
      fv[k] = decay_pow(zp[(long)t * ldz + h * d + k] + ldf(f_bias + h * d + k), inv_tau);
    } else {
      qv[k] = qz / (1.f + expf(-qz));
      const float lw = ldf(lower + h * d + k);
      const float fz = row[H * d + h * d + k] + ldf(f_bias + h * d + k);
      fv[k] = lw + (1.f - lw) / (1.f + expf(-fz));
    }
  }
  __syncthreads();
  const bool fresh = positions[t] == 0;
  float o = 0.f;
  if (c < dv) {
    float* sp = state + ((long)slot * H + h) * d * dv + c;
    const float v = row[2 * H * d + h * dv + c];
    int i = 0;
    for (; i + 8 <= d; i += 8) {          // 8 independent loads in flight per thread
      float old[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) old[u] = fresh ? 0.f : sp[(long)(i + u) * dv];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float fi = fv[i + u];
        const float sv = fi * old[u] + (GLA ? kv[i + u] : 1.f - fi) * v;
        sp[(long)(i + u) * dv] = sv;
        o += sv * qv[i + u];
      }
    }
    for (; i < d; ++i) {
      const float fi = fv[i];
      const float sv = fi * (fresh ? 0.f : sp[(long)i * dv]) + (GLA ? kv[i] : 1.f - fi) * v;
      sp[(long)i * dv] = sv;
      o += sv * qv[i];
    }
  }
  const float ss = block_sum(o * o, red);
  if (c < dv) {
    float val = o * (1.f / sqrtf(ss / (float)dv + eps)) * ldf(norm_w + c);
    if (GLA) val *= silu32(row[2 * H * d + H * dv + h * dv + c]);
    stf(out + (long)t * ldo + h * dv + c, val);
  }
}

}  // namespace

template <bool GLA>
static int launch_recurrence(const float* proj, int ldp, const void* f_bias, const void* lower,
                             const void* norm_w, float eps, float* state, const int* slots,
                             const int* cu, const int* positions, void* out, int ldo,
                             int num_seqs, int max_seqlen, int H, int d, int dv, int dt,
                             const float* zp, int ldz, float inv_tau, float qscale,
                             hipStream_t st) {
  if (num_seqs <= 0) return 0;
  const int threads = ((dv + 63) / 64) * 64;
  if (H < 1 || d < 1 || dv < 1 || threads > 1024) return (int)hipErrorInvalidValue;
  if (max_seqlen == 1) {                 // a decode step: stream the state, no LDS copy
    dim3 grid1(H, num_seqs);
    const size_t sh1 = ((size_t)(GLA ? 3 : 2) * d + 16) * 4;
    if (sh1 > 48 * 1024) return (int)hipErrorInvalidValue;
    if (dt == 0)
      hgrn2_step_kernel<u16, GLA><<<grid1, threads, sh1, st>>>(
          proj, ldp, (const u16*)f_bias, (const u16*)lower, (const u16*)norm_w, eps, state, slots,
          cu, positions, (u16*)out, ldo, H, d, dv, zp, ldz, inv_tau, qscale);
    else if (dt == 1)
      hgrn2_step_kernel<float, GLA><<<grid1, threads, sh1, st>>>(
          proj, ldp, (const float*)f_bias, (const float*)lower, (const float*)norm_w, eps, state,
          slots, cu, positions, (float*)out, ldo, H, d, dv, zp, ldz, inv_tau, qscale);
    else return (int)hipErrorInvalidValue;
    DLI_RETURN_LAUNCH();
  }
  // register form: d in {16, 32, 64, 128}, the state rows dealt to P thread groups
  int D = (d == 16 || d == 32 || d == 64 || d == 128) ? d : 0;
  const int P = D >= 64 ? 4 : (D == 32 ? 2 : 1);
  if (D && threads * P > 1024) D = 0;
  const int nthreads = D ? threads * P : threads;
  const size_t sh = ((size_t)(D ? 0 : d * dv) + (GLA ? 3 : 2) * TC * d +
                     (size_t)((D ? P : 1) + 1) * TC * dv) * 4;
  if (sh > 160 * 1024) return (int)hipErrorInvalidValue;
  dim3 grid(H, num_seqs);
#define HGRN2_LAUNCH(ST, DD, PP)                                                               \
  do {                                                                                         \
    if (sh > 48 * 1024) {                                                                      \
      hipError_t e = hipFuncSetAttribute((const void*)hgrn2_kernel<ST, DD, PP, GLA>,           \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh); \
      if (e != hipSuccess) return (int)e;                                                      \
    }                                                                                          \
    hgrn2_kernel<ST, DD, PP, GLA><<<grid, nthreads, sh, st>>>(                                 \
        proj, ldp, (const ST*)f_bias, (const ST*)lower, (const ST*)norm_w, eps, state, slots,  \
        cu, positions, (ST*)out, ldo, H, d, dv, zp, ldz, inv_tau, qscale);                     \
  } while (0)
#define HGRN2_BY_D(ST)                                   \
  do {                                                   \
    switch (D) {                                         \
      case 16: HGRN2_LAUNCH(ST, 16, 1); break;           \
      case 32: HGRN2_LAUNCH(ST, 32, 2); break;           \
      case 64: HGRN2_LAUNCH(ST, 64, 4); break;           \
      case 128: HGRN2_LAUNCH(ST, 128, 4); break;         \
      default: HGRN2_LAUNCH(ST, 0, 1); break;            \
    }                                                    \
  } while (0)
  if (dt == 0) HGRN2_BY_D(u16);
  else if (dt == 1) HGRN2_BY_D(float);
  else return (int)hipErrorInvalidValue;
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_hgrn2(const float* proj, int ldp, const void* f_bias, const void* lower,
                         const void* norm_w, float eps, float* state, const int* slots,
                         const int* cu, const int* positions, void* out, int ldo, int num_seqs,
                         int max_seqlen, int H, int d, int dv, int dt, hipStream_t st) {
  return launch_recurrence<false>(proj, ldp, f_bias, lower, norm_w, eps, state, slots, cu,
                                  positions, out, ldo, num_seqs, max_seqlen, H, d, dv, dt,
                                  nullptr, 0, 0.f, 0.f, st);
}

// Gated linear attention: proj row [H*d q | H*d k | H*dv v | H*dv gate | ...] (fp32), z
// [T, H*d] (fp32) the decay's pre-activation, a_bias its bias, inv_tau = 1 / tau.
extern "C" int dli_gla(const float* proj, int ldp, const float* z, int ldz, const void* a_bias,
                       float inv_tau, float qscale, const void* norm_w, float eps, float* state,
                       const int* slots, const int* cu, const int* positions, void* out, int ldo,
                       int num_seqs, int max_seqlen, int H, int d, int dv, int dt,
                       hipStream_t st) {
  if (z == nullptr || a_bias == nullptr) return (int)hipErrorInvalidValue;
  return launch_recurrence<true>(proj, ldp, a_bias, nullptr, norm_w, eps, state, slots, cu,
                                 positions, out, ldo, num_seqs, max_seqlen, H, d, dv, dt, z, ldz,
                                 inv_tau, qscale, st);
}
