// Sliding-window attention over a token-major paged cache, for every step kind at once: a
// step's query tokens (whole prompts, portions of prompts, single decoded tokens, mixed) first
// write their keys / values into the cache, then each query attends the cached positions
// [max(0, p - window + 1), p] of its own sequence through the block table.
//
// Options, each a parameter so that several designs share the kernel:
//  * slopes  != null: score -= slope[h] * (p - j)  (linear distance bias)
//  * talk    != null: after the softmax the heads' weights are mixed,
//                     w'[h][j] = sum_g talk[h][g] w[g][j]; head h applies w' to the values of its
//                     own key/value head. Needs the normalised weights of every head, so the
//                     kernel makes two passes over the window: (1) running max / sum per head,
//                     (2) weights, mix, weighted value sum.
//  * gate    != null: out *= sigmoid(gate) (fp32 pre-activation of the same token, ldg); with
//                     head_gate the gate row holds one number per head
//  * sink    != null: exp(sink[h]) joins head h's softmax denominator: a key with that score
//                     and no value, counted once (the running max / sum start from it)
//  * out_scale:       the output is multiplied by it
//  * chunk   > 0: a query also sees only the keys of its own block of `chunk` positions
//                     (blocks counted from position 0 of the sequence)
//  * Gk != G: the key rows hold Gk heads of dq while the values hold G heads of dv (Gk = 1:
//                     every query head scores the whole key row — head mixing before the
//                     softmax folded into the queries)
//  * dq != dv, and v_cache may alias k_cache with its own row stride: latent attention in the
//    absorbed form reads one [latent | rotated key] row per token, scores over all of it and
//    values = its first dv columns (G = 1: every head shares the row).
//
// Cache rows: k row of slot s, kv head g at k_cache + s * k_stride + g * dq (v likewise with
// dv). Scores, softmax, mixing and the value sum are fp32 for both storage types.
//
// This is the scalar form (one workgroup per query token, heads x keys spread over the
// threads); the MFMA form for bf16 tiles queries and is selected by the launcher when the
// shapes fit it.
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

constexpr int KT = 64;          // keys per tile
constexpr int MAX_ACC = 64;     // output elements per thread: H * dv <= 256 * MAX_ACC

struct WinAttnArgs {
  const void* q; int ldq;               // [T, H, dq]
  const void* k; long k_stride;         // cache rows
  const void* v; long v_stride;
  void* out; int ldo;                   // [T, H, dv]
  const float* gate; int ldg;           // [T, H*dv] fp32 or null
  const float* slopes;                  // [H] or null
  const float* talk;                    // [H, H] or null
  const int* cu; const int* positions;  // [S+1], [T]
  const int* block_tables; int bt_stride; int block_size;
  int H, G, dq, dv, window;
  float scale;
  int Gk, chunk;
  const float* sink;                    // [H] or null
  int head_gate; float out_scale;
};

template <typename S>
__global__ void __launch_bounds__(256) window_attention_kernel(WinAttnArgs a) {
  extern __shared__ float sm[];
  const int H = a.H, G = a.G, dq = a.dq, dv = a.dv;
  float* qs = sm;                        // [H * dq]
  float* pt = qs + H * dq;               // [H][KT] scores / weights
  float* mx = pt + H * KT;               // [H][KT] mixed weights
  float* hm = mx + H * KT;               // [H] running max
  float* hl = hm + H;                    // [H] running sum
  int* slot = (int*)(hl + H);            // [KT]
  const int s = blockIdx.y;
  const int t = a.cu[s] + blockIdx.x;
  if (t >= a.cu[s + 1]) return;
  const int p = a.positions[t];
  int lo = max(0, p - a.window + 1);
  if (a.chunk > 0) lo = max(lo, p / a.chunk * a.chunk);
  const int n = p + 1 - lo;
  const int tid = threadIdx.x;
  const S* qrow = (const S*)a.q + (long)t * a.ldq;
  for (int i = tid; i < H * dq; i += blockDim.x) qs[i] = ldf(qrow + i);
  for (int h = tid; h < H; h += blockDim.x) {
    hm[h] = a.sink != nullptr ? a.sink[h] : -INFINITY;
    hl[h] = a.sink != nullptr ? 1.f : 0.f;
  }
  const int* bt = a.block_tables + (long)s * a.bt_stride;
  const int hpg = H / G, hpk = H / a.Gk;
  float acc[MAX_ACC];
#pragma unroll
  for (int i = 0; i < MAX_ACC; ++i) acc[i] = 0.f;
  const int ntiles = (n + KT - 1) / KT;

  for (int pass = 0; pass < 2; ++pass) {
    for (int tile = 0; tile < ntiles; ++tile) {
      const int j0 = lo + tile * KT;
      __syncthreads();
      if (tid < KT) {
        const int j = j0 + tid;
        slot[tid] = j <= p ? bt[j / a.block_size] * a.block_size + j % a.block_size : -1;
      }
      __syncthreads();
      for (int idx = tid; idx < H * KT; idx += blockDim.x) {
        const int h = idx / KT, jj = idx % KT;
        const int sl = slot[jj];
        float sc = -INFINITY;
        if (sl >= 0) {
          const S* kr = (const S*)a.k + (long)sl * a.k_stride + (h / hpk) * dq;
          const float* qh = qs + h * dq;
          float d0 = 0.f;
          for (int c = 0; c < dq; ++c) d0 += qh[c] * ldf(kr + c);
          sc = d0 * a.scale;
          if (a.slopes != nullptr) sc -= a.slopes[h] * (float)(p - (j0 + jj));
        }
        pt[idx] = sc;
      }
      __syncthreads();
      if (pass == 0) {
        // one wave per head in turn: tile max and sum folded into the running pair
        const int lane = tid & 63, wid = tid >> 6, nw = blockDim.x >> 6;
        for (int h = wid; h < H; h += nw) {
          const float sc = pt[h * KT + lane];
          const float m_old = hm[h];
          const float m_new = fmaxf(m_old, wave_max(sc));
          const float e = sc == -INFINITY ? 0.f : expf(sc - m_new);
          const float sum = wave_sum(e);
          if (lane == 0) {
            hl[h] = (m_old == -INFINITY ? 0.f : hl[h] * expf(m_old - m_new)) + sum;
            hm[h] = m_new;
          }
        }
      } else {
        for (int idx = tid; idx < H * KT; idx += blockDim.x) {
          const int h = idx / KT;
          const float sc = pt[idx];
          pt[idx] = sc == -INFINITY ? 0.f : expf(sc - hm[h]) / hl[h];
        }
        __syncthreads();
        const float* wts = pt;
        if (a.talk != nullptr) {
          for (int idx = tid; idx < H * KT; idx += blockDim.x) {
            const int h = idx / KT, jj = idx % KT;
            float m = 0.f;
            for (int g = 0; g < H; ++g) m += a.talk[h * H + g] * pt[g * KT + jj];
            mx[idx] = m;
          }
          __syncthreads();
          wts = mx;
        }
        const int kmax = min(KT, p + 1 - j0);
#pragma unroll
        for (int i = 0; i < MAX_ACC; ++i) {
          const int o = tid + i * 256;
          if (o < H * dv) {
            const int h = o / dv, c = o % dv;
            const S* vb = (const S*)a.v + (h / hpg) * dv + c;
            const float* wh = wts + h * KT;
            float sum = acc[i];
            for (int jj = 0; jj < kmax; ++jj) sum += wh[jj] * ldf(vb + (long)slot[jj] * a.v_stride);
            acc[i] = sum;
          }
        }
      }
    }
  }
  S* orow = (S*)a.out + (long)t * a.ldo;
#pragma unroll
  for (int i = 0; i < MAX_ACC; ++i) {
    const int o = tid + i * 256;
    if (o < H * dv) {
      float v = acc[i];
      if (a.gate != nullptr)
        v *= 1.f / (1.f + expf(-a.gate[(long)t * a.ldg + (a.head_gate ? o / dv : o)]));
      stf(orow + o, v * a.out_scale);
    }
  }
}

}  // namespace

extern "C" int dli_window_attention(
    const void* q, int ldq, const void* k, long k_stride, const void* v, long v_stride, void* out,
    int ldo, const float* gate, int ldg, const float* slopes, const float* talk, const int* cu,
    const int* positions, const int* block_tables, int bt_stride, int block_size, int num_seqs,
    int max_seqlen, int H, int G, int dq, int dv, int window, float scale, int Gk, int chunk,
    const float* sink, int head_gate, float out_scale, int dt, hipStream_t st) {
  if (num_seqs <= 0 || max_seqlen <= 0) return 0;
  if (H < 1 || G < 1 || H % G || Gk < 1 || H % Gk || chunk < 0 || dq < 1 || dv < 1 ||
      window < 1 || block_size < 1 ||
      (long)H * dv > 256L * MAX_ACC)
    return (int)hipErrorInvalidValue;
  const size_t sh = ((size_t)H * dq + 2 * (size_t)H * KT + 2 * H + KT) * 4;
  if (sh > 160 * 1024) return (int)hipErrorInvalidValue;
  if (sh > 48 * 1024) {                   // opt in to the large LDS carve-out once per type
    static bool raised[2] = {false, false};
    if (dt >= 0 && dt < 2 && !raised[dt]) {
      const void* fn = dt == 0 ? (const void*)window_attention_kernel<u16>
                               : (const void*)window_attention_kernel<float>;
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         160 * 1024);
      if (e != hipSuccess) return (int)e;
      raised[dt] = true;
    }
  }
  WinAttnArgs a{q, ldq, k, k_stride, v, v_stride, out, ldo, gate, ldg, slopes, talk, cu,
                positions, block_tables, bt_stride, block_size, H, G, dq, dv, window, scale,
                Gk, chunk, sink, head_gate, out_scale};
  dim3 grid(max_seqlen, num_seqs);
  if (dt == 0) window_attention_kernel<u16><<<grid, 256, sh, st>>>(a);
  else if (dt == 1) window_attention_kernel<float><<<grid, 256, sh, st>>>(a);
  else return (int)hipErrorInvalidValue;
  DLI_RETURN_LAUNCH();
}
