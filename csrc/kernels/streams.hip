// Row kernels of the hyper-connected designs (models/hybrid.py, ops/hybrid.py). S = storage
// type (u16 = bf16 bits, or float); the streams, norms and sums are fp32.
//
//  * hyper_mix     hyper-connections over ns copies of the residual stream, xs [T, ns, dim]:
//                  with a finished sublayer's output y and its vector prev = [read | write |
//                  mix] (ns + ns + ns*ns floats, mix indexed [from, to]) every stream becomes
//                      xs[r] = sum_s mix[s][r] xs[s] + write[r] * y          (all r at once)
//                  and with the next sublayer's read weights the row u = sum_s read[s] xs[s]
//                  leaves RMS-normed times (w + w_offset) as S, or as it is in fp32 (w null).
//                  One launch does a sublayer's write-back and the next one's read + norm.
//  * sink_prepare  q / k RMS-normed over their whole rows (all heads at once) with a weight
//                  per column, the first rot_dims dims of every head rotated (dimension i with
//                  i + rot_dims/2; angle = position * freq[i] formed in double; cos and sin
//                  times mscale), k and v -> cache rows, q -> S
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

constexpr int MAXS = 8;          // streams

// One workgroup per token (256 threads; 1024 for the few wide rows of a decode step, which
// are bound by latency). VEC = 4: 16-byte accesses of the fp32 rows (dim % 4 == 0).
template <typename S, int VEC>
__global__ void __launch_bounds__(1024) hyper_mix_kernel(
    float* __restrict__ xs, const float* __restrict__ y, int ldy, const float* __restrict__ prev,
    const float* __restrict__ read, const S* __restrict__ w, void* __restrict__ h, int ns,
    int dim, float eps, float w_offset) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  float* urow = sm;                        // [dim]
  float* red = urow + dim;                 // [16]
  float* cf = red + 16;                    // [ns*(ns+2)] prev, then [ns] read
  const int t = blockIdx.x;
  const int nc = ns * (ns + 2);
  float* xr = xs + (long)t * ns * dim;
  for (int i = threadIdx.x; i < nc + ns; i += blockDim.x)
    cf[i] = i < nc ? (prev != nullptr ? prev[i] : 0.f) : (read != nullptr ? read[i - nc] : 0.f);
  __syncthreads();
  const float* wr = cf + ns;               // write weights
  const float* mix = cf + 2 * ns;          // [from][to]
  const float* rd = cf + nc;
  float ss = 0.f;
  for (int c = threadIdx.x * VEC; c < dim; c += blockDim.x * VEC) {
    float x[MAXS][VEC];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
      if (s < ns) {
        if (VEC == 4) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(xr + (long)s * dim + c);
#pragma unroll
          for (int u = 0; u < VEC; ++u) x[s][u] = v[u];
        } else {
          x[s][0] = xr[(long)s * dim + c];
        }
      }
    }
    if (y != nullptr) {
      float yv[VEC], nx[MAXS][VEC];
#pragma unroll
      for (int u = 0; u < VEC; ++u) yv[u] = y[(long)t * ldy + c + u];
#pragma unroll
      for (int r = 0; r < MAXS; ++r) {
        if (r < ns) {
#pragma unroll
          for (int u = 0; u < VEC; ++u) {
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < MAXS; ++s)
              if (s < ns) acc += mix[s * ns + r] * x[s][u];
            nx[r][u] = acc + wr[r] * yv[u];
          }
          if (VEC == 4)
            *reinterpret_cast<f32x4*>(xr + (long)r * dim + c) =
                f32x4{nx[r][0], nx[r][VEC > 1 ? 1 : 0], nx[r][VEC > 2 ? 2 : 0], nx[r][VEC > 3 ? 3 : 0]};
          else
            xr[(long)r * dim + c] = nx[r][0];
        }
      }
#pragma unroll
      for (int r = 0; r < MAXS; ++r)
        if (r < ns) {
#pragma unroll
          for (int u = 0; u < VEC; ++u) x[r][u] = nx[r][u];
        }
    }
    if (read != nullptr) {
#pragma unroll
      for (int u = 0; u < VEC; ++u) {
        float acc = 0.f;
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
          if (s < ns) acc += rd[s] * x[s][u];
        if (w == nullptr) ((float*)h)[(long)t * dim + c + u] = acc;
        else urow[c + u] = acc;
        ss += acc * acc;
      }
    }
  }
  if (read == nullptr || w == nullptr) return;
  const float tot = block_sum(ss, red);
  const float rs = 1.f / sqrtf(tot / (float)dim + eps);
  for (int c = threadIdx.x; c < dim; c += blockDim.x)
    stf((S*)h + (long)t * dim + c, urow[c] * rs * (ldf(w + c) + w_offset));
}

// One workgroup per token. proj row (fp32): [H*d q | G*d k | G*dv v | ...].
template <typename S>
__global__ void __launch_bounds__(1024) sink_prepare_kernel(
    const float* __restrict__ proj, int ldp, const S* __restrict__ qw, const S* __restrict__ kw,
    float eps, int H, int G, int d, int dv, int rot, const double* __restrict__ freq,
    float mscale, const int* __restrict__ positions, S* __restrict__ q_out,
    S* __restrict__ kcache, S* __restrict__ vcache, const int* __restrict__ slots) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int nq = H * d, nk = G * d, hr = rot >> 1;
  float* row = sm;                         // [nq + nk] normed q | k
  float* cs = row + nq + nk;               // [rot / 2]
  float* sn = cs + hr;                     // [rot / 2]
  float* red = sn + hr;                    // [16]
  const int t = blockIdx.x;
  const float* pr = proj + (long)t * ldp;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < nq + nk; c += blockDim.x) {
    const float v = pr[c];
    row[c] = v;
    if (c < nq) sq += v * v; else sk += v * v;
  }
  const double pos = (double)positions[t];
  for (int i = threadIdx.x; i < hr; i += blockDim.x) {
    const double a = pos * freq[i];
    cs[i] = (float)(cos(a) * (double)mscale);
    sn[i] = (float)(sin(a) * (double)mscale);
  }
  const float tq = block_sum(sq, red);
  const float tk = block_sum(sk, red);
  const float rq = 1.f / sqrtf(tq / (float)nq + eps), rk = 1.f / sqrtf(tk / (float)nk + eps);
  for (int c = threadIdx.x; c < nq + nk; c += blockDim.x)
    row[c] = c < nq ? row[c] * rq * ldf(qw + c) : row[c] * rk * ldf(kw + c - nq);
  __syncthreads();
  const int slot = slots[t];
  for (int c = threadIdx.x; c < nq + nk; c += blockDim.x) {
    const int j = (c < nq ? c : c - nq) % d;
    float v = row[c];
    if (j < rot) {
      const bool second = j >= hr;
      const int i = second ? j - hr : j;
      const float other = row[second ? c - hr : c + hr];
      v = second ? v * cs[i] + other * sn[i] : v * cs[i] - other * sn[i];
    }
    if (c < nq) stf(q_out + (long)t * nq + c, v);
    else if (slot >= 0) stf(kcache + (long)slot * nk + (c - nq), v);
  }
  if (slot >= 0)
    for (int c = threadIdx.x; c < G * dv; c += blockDim.x)
      stf(vcache + (long)slot * G * dv + c, pr[nq + nk + c]);
}

}  // namespace

#define DT_SWITCH2(dt, A, B)                      \
  do {                                            \
    if ((dt) == 0) { A; }                         \
    else if ((dt) == 1) { B; }                    \
    else return (int)hipErrorInvalidValue;        \
  } while (0)

extern "C" int dli_hyper_mix(float* xs, const float* y, int ldy, const float* prev,
                             const float* read, const void* w, void* h, int T, int ns, int dim,
                             float eps, float w_offset, int dt, hipStream_t st) {
  if (T <= 0) return 0;
  if (ns < 1 || ns > MAXS || dim < 1 || (y != nullptr) != (prev != nullptr) ||
      (read != nullptr && h == nullptr) || (read == nullptr && y == nullptr))
    return (int)hipErrorInvalidValue;
  const size_t sh = ((size_t)dim + 16 + (size_t)ns * (ns + 3)) * 4;
  if (sh > 60000) return (int)hipErrorInvalidValue;
  const bool v4 = dim % 4 == 0 && (uintptr_t)xs % 16 == 0 &&
                  (y == nullptr || ((uintptr_t)y % 16 == 0 && ldy % 4 == 0));
  const int nt = (T <= 1024 && dim >= 2048) ? 1024 : 256;
#define HM_LAUNCH(S, V)                                                                       \
  hyper_mix_kernel<S, V><<<T, nt, sh, st>>>(xs, y, ldy, prev, read, (const S*)w, h, ns, dim,  \
                                            eps, w_offset)
  if (v4) DT_SWITCH2(dt, HM_LAUNCH(u16, 4), HM_LAUNCH(float, 4));
  else DT_SWITCH2(dt, HM_LAUNCH(u16, 1), HM_LAUNCH(float, 1));
#undef HM_LAUNCH
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_sink_prepare(const float* proj, int ldp, const void* qw, const void* kw,
                                float eps, int T, int H, int G, int d, int dv, int rot_dims,
                                const double* freq, float mscale, const int* positions,
                                void* q_out, void* kcache, void* vcache, const int* slots, int dt,
                                hipStream_t st) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || H % G || d < 1 || dv < 1 || rot_dims < 0 || (rot_dims & 1) ||
      rot_dims > d || (rot_dims > 0 && freq == nullptr))
    return (int)hipErrorInvalidValue;
  const size_t sh = ((size_t)(H + G) * d + rot_dims + 16) * 4;
  if (sh > 60000) return (int)hipErrorInvalidValue;
  const int nt = (T <= 1024 && (H + G) * d >= 2048) ? 1024 : 256;
  DT_SWITCH2(dt,
             (sink_prepare_kernel<u16><<<T, nt, sh, st>>>(
                 proj, ldp, (const u16*)qw, (const u16*)kw, eps, H, G, d, dv, rot_dims, freq,
                 mscale, positions, (u16*)q_out, (u16*)kcache, (u16*)vcache, slots)),
             (sink_prepare_kernel<float><<<T, nt, sh, st>>>(
                 proj, ldp, (const float*)qw, (const float*)kw, eps, H, G, d, dv, rot_dims, freq,
                 mscale, positions, (float*)q_out, (float*)kcache, (float*)vcache, slots)));
  DLI_RETURN_LAUNCH();
}
