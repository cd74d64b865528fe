// Row kernels of post-norm layer-list designs: the residual stream x is fp32; every sublayer
// reads x itself (its rounding to the storage type S feeds the GEMMs), and a layer norm with
// weight and bias follows each sum. S is bf16 (dt = 0) or fp32 (dt = 1); all arithmetic is fp32.
//
//  * prev_tokens       the token before every row of a step (the row above, the sequence's
//                      state slot for a portion's first row, -1 at position 0); the slot then
//                      takes the portion's last token
//  * embedding_bigram  x = table[id] + bigram[(prev * mul_prev + id * mul_cur) mod buckets]
//                      (row `buckets` when there is no previous token), fp32 and S copies
//  * postnorm          x = LayerNorm(keep * x + y) * w + b in place, and its S copy; with a row
//                      list: those rows only, S out, x untouched (the final norm)
//  * add_rmsnormed     x += y / sqrt(mean(y^2) + eps) * w in place, and the S copy of x
//  * side_gate         gelu_tanh(gate) * table[id, col0 + c] -> S (a per-layer slice of a
//                      second embedding table gates a small projection)
//  * rmsnorm_cols      RMS norm * w (* sigmoid(gate)) of a column slice of an fp32 projection -> S
//  * latent_prepare    latent attention with the queries and the compressed kv in separate
//                      projections: RMS norm of the latent -> cache, rotary on the shared key ->
//                      cache (skipped by a layer that reads another layer's cache), rotary on
//                      every head's rotated query part, either pair layout
//  * head_gate         o[t, h, :] * sigmoid(g[t, h]) -> S
//  * logit_router      fp32 logits h . W + b, the `top` largest, softmax over the chosen
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

// four consecutive elements (16-byte aligned fp32, 8-byte aligned bf16)
template <typename S> __device__ __forceinline__ f32x4 ld4(const S* p);
template <> __device__ __forceinline__ f32x4 ld4<float>(const float* p) {
  return *reinterpret_cast<const f32x4*>(p);
}
template <> __device__ __forceinline__ f32x4 ld4<u16>(const u16* p) {
  const uint2 b = *reinterpret_cast<const uint2*>(p);
  return f32x4{__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xffff0000u),
               __uint_as_float(b.y << 16), __uint_as_float(b.y & 0xffff0000u)};
}
template <typename S> __device__ __forceinline__ void st4(S* p, f32x4 v);
template <> __device__ __forceinline__ void st4<float>(float* p, f32x4 v) {
  *reinterpret_cast<f32x4*>(p) = v;
}
template <> __device__ __forceinline__ void st4<u16>(u16* p, f32x4 v) {
  uint2 pk;
  pk.x = pack2bf(v[0], v[1]);
  pk.y = pack2bf(v[2], v[3]);
  *reinterpret_cast<uint2*>(p) = pk;
}

// Grid: one workgroup per sequence. Every row's predecessor is read before the slot is
// overwritten (the barrier), so a one-token portion sees the token of the step before.
__global__ void __launch_bounds__(256) prev_tokens_kernel(
    int* __restrict__ prev, const int* __restrict__ ids, int* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ cu,
    const int* __restrict__ positions) {
  const int s = blockIdx.x;
  const int t0 = cu[s], t1 = cu[s + 1];
  if (t1 <= t0) return;
  const int slot = slots != nullptr ? slots[s] : -1;
  for (int t = t0 + threadIdx.x; t < t1; t += blockDim.x) {
    int p;
    if (t > t0) p = ids[t - 1];
    else p = (positions[t0] == 0 || slot < 0) ? -1 : state[slot];
    prev[t] = p;
  }
  __syncthreads();
  if (threadIdx.x == 0 && slot >= 0) state[slot] = ids[t1 - 1];
}

template <typename S>
__global__ void __launch_bounds__(256) embedding_bigram_kernel(
    float* __restrict__ x, S* __restrict__ xs, const int* __restrict__ ids,
    const int* __restrict__ prev, const S* __restrict__ table, const S* __restrict__ bigram,
    int T, int dim, int vocab, int buckets, long mul_prev, long mul_cur) {
  const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long)T * dim) return;
  const int t = (int)(gid / dim), c = (int)(gid % dim);
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  float v = ldf(table + (long)id * dim + c);
  if (bigram != nullptr) {
    const int p = prev[t];
    long row = buckets;                        // no previous token: the table's last row
    if (p >= 0) {
      row = ((long)p * mul_prev + (long)id * mul_cur) % buckets;
      if (row < 0) row += buckets;
    }
    v += ldf(bigram + row * dim + c);
  }
  x[gid] = v;
  stf(xs + gid, v);
}

// One workgroup per row: v = keep * x + y; mean and variance (of the deviations, two passes
// over the row held in LDS); x = (v - mean) * rsqrt(var + eps) * w + b.
template <typename S>
__global__ void __launch_bounds__(256) postnorm_kernel(
    float* __restrict__ x, const float* __restrict__ y, int ldy, float keep,
    const S* __restrict__ w, const S* __restrict__ b, S* __restrict__ h, int dim, float eps,
    const long* __restrict__ rows_idx, bool vec4) {
  extern __shared__ __attribute__((aligned(16))) float row[];   // dim floats + 16 reduction slots
  float* red = row + dim;
  const int r = blockIdx.x;
  const long src = rows_idx ? rows_idx[r] : r;
  float* xr = x + src * dim;
  float s = 0.f;
  if (vec4) {                                    // 16-byte loads and stores of the rows
    for (int c = threadIdx.x * 4; c < dim; c += blockDim.x * 4) {
      f32x4 v = *reinterpret_cast<const f32x4*>(xr + c);
      if (rows_idx == nullptr) {
        v *= keep;
        if (y != nullptr) v += *reinterpret_cast<const f32x4*>(y + (long)r * ldy + c);
      }
      *reinterpret_cast<f32x4*>(row + c) = v;
      s += (v[0] + v[1]) + (v[2] + v[3]);
    }
    const float mean = block_sum(s, red) / (float)dim;
    float q = 0.f;
    for (int c = threadIdx.x * 4; c < dim; c += blockDim.x * 4) {
      const f32x4 d = *reinterpret_cast<const f32x4*>(row + c) - mean;
      q += (d[0] * d[0] + d[1] * d[1]) + (d[2] * d[2] + d[3] * d[3]);
    }
    const float rs = 1.f / sqrtf(block_sum(q, red) / (float)dim + eps);
    for (int c = threadIdx.x * 4; c < dim; c += blockDim.x * 4) {
      const f32x4 v = (*reinterpret_cast<const f32x4*>(row + c) - mean) * rs * ld4(w + c) +
                      ld4(b + c);
      if (rows_idx == nullptr) *reinterpret_cast<f32x4*>(xr + c) = v;
      st4(h + (long)r * dim + c, v);
    }
    return;
  }
  for (int c = threadIdx.x; c < dim; c += blockDim.x) {
    float v = xr[c];
    if (rows_idx == nullptr) {
      v *= keep;
      if (y != nullptr) v += y[(long)r * ldy + c];
    }
    row[c] = v;
    s += v;
  }
  const float mean = block_sum(s, red) / (float)dim;
  float q = 0.f;
  for (int c = threadIdx.x; c < dim; c += blockDim.x) { const float d = row[c] - mean; q += d * d; }
  __syncthreads();                               // red is reused
  const float rs = 1.f / sqrtf(block_sum(q, red) / (float)dim + eps);
  for (int c = threadIdx.x; c < dim; c += blockDim.x) {
    const float v = (row[c] - mean) * rs * ldf(w + c) + ldf(b + c);
    if (rows_idx == nullptr) xr[c] = v;
    stf(h + (long)r * dim + c, v);
  }
}

template <typename S>
__global__ void __launch_bounds__(256) add_rmsnormed_kernel(
    float* __restrict__ x, const float* __restrict__ y, int ldy, const S* __restrict__ w,
    S* __restrict__ h, int dim, float eps, bool vec4) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const float* yr = y + (long)r * ldy;
  float s = 0.f;
  if (vec4) {
    for (int c = threadIdx.x * 4; c < dim; c += blockDim.x * 4) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(yr + c);
      s += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
    }
    const float rs = 1.f / sqrtf(block_sum(s, red) / (float)dim + eps);
    for (int c = threadIdx.x * 4; c < dim; c += blockDim.x * 4) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(x + (long)r * dim + c) +
                      *reinterpret_cast<const f32x4*>(yr + c) * rs * ld4(w + c);
      *reinterpret_cast<f32x4*>(x + (long)r * dim + c) = v;
      st4(h + (long)r * dim + c, v);
    }
    return;
  }
  for (int c = threadIdx.x; c < dim; c += blockDim.x) { const float v = yr[c]; s += v * v; }
  const float rs = 1.f / sqrtf(block_sum(s, red) / (float)dim + eps);
  for (int c = threadIdx.x; c < dim; c += blockDim.x) {
    const float v = x[(long)r * dim + c] + yr[c] * rs * ldf(w + c);
    x[(long)r * dim + c] = v;
    stf(h + (long)r * dim + c, v);
  }
}

__device__ __forceinline__ float gelu_tanh32(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename S>
__global__ void __launch_bounds__(256) side_gate_kernel(
    S* __restrict__ out, const float* __restrict__ gate, int ldg, const int* __restrict__ ids,
    const S* __restrict__ table, int ldt, int col0, int T, int n, int vocab) {
  const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long)T * n) return;
  const int t = (int)(gid / n), c = (int)(gid % n);
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  stf(out + gid, gelu_tanh32(gate[(long)t * ldg + c]) * ldf(table + (long)id * ldt + col0 + c));
}

// One wave per row.
template <typename S>
__global__ void __launch_bounds__(256) rmsnorm_cols_kernel(
    S* __restrict__ out, const float* __restrict__ src, int lds, const S* __restrict__ w, int T,
    int n, float eps, bool vec4, const float* __restrict__ gate, int ldg, int groups, int ldo,
    float out_scale) {
  // a row = one of `groups` parts (n wide each, normed by itself) of a token's row
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= T * groups) return;
  const int t = row / groups, go = (row % groups) * n;
  const float* r = src + (long)t * lds + go;
  w += go;
  out += (long)t * ldo + go;
  if (gate != nullptr) gate += (long)t * ldg + go;
  float s = 0.f;
  if (vec4) {                                   // 16-byte loads, 4 columns a lane
    for (int c = lane * 4; c < n; c += 256) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(r + c);
      s += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
    }
    s = wave_sum(s);
    const float rs = 1.f / sqrtf(s / (float)n + eps);
    for (int c = lane * 4; c < n; c += 256) {
      f32x4 v = *reinterpret_cast<const f32x4*>(r + c) * rs * ld4(w + c);
      if (gate != nullptr) {
        const f32x4 g = *reinterpret_cast<const f32x4*>(gate + c);
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] *= 1.f / (1.f + expf(-g[u]));
      }
      st4(out + c, v * out_scale);
    }
    return;
  }
  for (int c = lane; c < n; c += 64) { const float v = r[c]; s += v * v; }
  s = wave_sum(s);
  const float rs = 1.f / sqrtf(s / (float)n + eps);
  for (int c = lane; c < n; c += 64) {
    float v = r[c] * rs * ldf(w + c);
    if (gate != nullptr) v *= 1.f / (1.f + expf(-gate[c]));
    stf(out + c, v * out_scale);
  }
}

// The same for few, wide rows (a decode step): one workgroup per row instead of one wave.
template <typename S>
__global__ void __launch_bounds__(256) rmsnorm_cols_block_kernel(
    S* __restrict__ out, const float* __restrict__ src, int lds, const S* __restrict__ w, int n,
    float eps, const float* __restrict__ gate, int ldg, int groups, int ldo, float out_scale) {
  __shared__ float red[16];
  const int t = blockIdx.x / groups, go = (blockIdx.x % groups) * n;
  const float* r = src + (long)t * lds + go;
  float s = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) { const float v = r[c]; s += v * v; }
  s = block_sum(s, red);
  const float rs = 1.f / sqrtf(s / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    float v = r[c] * rs * ldf(w + go + c);
    if (gate != nullptr) v *= 1.f / (1.f + expf(-gate[(long)t * ldg + go + c]));
    stf(out + (long)t * ldo + go + c, v * out_scale);
  }
}

// The rotation of element c of a rotated part `v` (length >= rot_dims): with `half` dimension
// i < rot_dims/2 pairs with i + rot_dims/2, else pairs are (2i, 2i+1). The pair (u, v) at angle
// a becomes (u cos a - v sin a, v cos a + u sin a); the angle position * frequency is formed in
// double and rounded once.
// `cs` / `sn` [rot_dims / 2]: this token's cosines and sines (LDS).
__device__ __forceinline__ float rotate_elem(const float* v, int c, int rot_dims, bool half,
                                             const float* cs, const float* sn) {
  if (c >= rot_dims) return v[c];
  const int hd = rot_dims >> 1;
  const int i = half ? (c < hd ? c : c - hd) : (c >> 1);
  const bool second = half ? c >= hd : (c & 1);
  const int partner = half ? (second ? c - hd : c + hd) : (c ^ 1);
  return second ? v[c] * cs[i] + v[partner] * sn[i] : v[c] * cs[i] - v[partner] * sn[i];
}

// Grid: one workgroup per token. qproj row (fp32): H heads of [d unrotated | dr rotated].
// kvproj row (fp32, nullable): [r latent | dr shared key]; the normed latent and the rotated key
// go to cache row `slot` (S, width r + dr). q_nope [T, H, d] (S) feeds the per-head absorb
// GEMM; q_full [T, H, r + dr] (S) receives the rotated tail [r, r + dr) of every head.
template <typename S>
__global__ void __launch_bounds__(256) latent_prepare_kernel(
    const float* __restrict__ qproj, int ldq, const float* __restrict__ kvproj, int ldkv,
    const S* __restrict__ cw, float eps, int H, int d, int dr, int r, int rot_dims,
    const double* __restrict__ inv_freq, const int* __restrict__ positions,
    const int* __restrict__ slots, S* __restrict__ q_nope, S* __restrict__ q_full,
    S* __restrict__ cache, bool half) {
  __shared__ float red[16];
  extern __shared__ float trig[];               // [rot_dims / 2] cosines, then sines
  float* cs = trig;
  float* sn = trig + (rot_dims >> 1);
  const int t = blockIdx.x;
  const double pos = (double)positions[t];
  for (int i = threadIdx.x; i < (rot_dims >> 1); i += blockDim.x) {
    const double a = pos * inv_freq[i];         // the angle in double, rounded once
    cs[i] = (float)cos(a);
    sn[i] = (float)sin(a);
  }
  __syncthreads();
  if (kvproj != nullptr) {
    const float* dkv = kvproj + (long)t * ldkv;
    const int slot = slots[t];
    float s = 0.f;
    for (int c = threadIdx.x; c < r; c += blockDim.x) { const float v = dkv[c]; s += v * v; }
    s = block_sum(s, red);
    const float rs = 1.f / sqrtf(s / (float)r + eps);
    if (slot >= 0) {
      S* cr = cache + (long)slot * (r + dr);
      for (int c = threadIdx.x; c < r; c += blockDim.x) stf(cr + c, dkv[c] * rs * ldf(cw + c));
      for (int c = threadIdx.x; c < dr; c += blockDim.x)
        stf(cr + r + c, rotate_elem(dkv + r, c, rot_dims, half, cs, sn));
    }
  }
  const float* row = qproj + (long)t * ldq;
  for (int i = threadIdx.x; i < H * (d + dr); i += blockDim.x) {
    const int h = i / (d + dr), c = i % (d + dr);
    if (c < d) {
      stf(q_nope + ((long)t * H + h) * d + c, row[i]);
    } else {
      stf(q_full + ((long)t * H + h) * (r + dr) + r + (c - d),
          rotate_elem(row + h * (d + dr) + d, c - d, rot_dims, half, cs, sn));
    }
  }
}

template <typename S>
__global__ void __launch_bounds__(256) head_gate_kernel(
    S* __restrict__ out, const float* __restrict__ o, const float* __restrict__ g, int ldg, int T,
    int H, int n) {
  const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long)T * H * n) return;
  const int t = (int)(gid / ((long)H * n)), h = (int)((gid / n) % H);
  stf(out + gid, o[gid] / (1.f + expf(-g[(long)t * ldg + h])));
}

constexpr int ROUTER_MAX = 1024;

// Grid: one workgroup per token. The row is staged in LDS as fp32; every wave takes experts in
// turn; thread 0 then picks the `top` largest logits (the lowest index wins a tie) and weighs
// them by the softmax over the chosen ones. A row of NaNs still selects valid ids.
template <typename S>
__global__ void __launch_bounds__(256) logit_router_kernel(
    float* __restrict__ topk_w, int* __restrict__ topk_ids, const S* __restrict__ h, int ldh,
    const S* __restrict__ W, const float* __restrict__ bias, int D, int n, int top, bool vec) {
  extern __shared__ __attribute__((aligned(16))) float rsm[];   // [D] row, [n] logits
  float* row = rsm;
  float* z = rsm + D;
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int c = threadIdx.x; c < D; c += blockDim.x) row[c] = ldf(h + (long)t * ldh + c);
  __syncthreads();
  constexpr int CH = 16 / sizeof(S);            // elements of a 16-byte load
  const int nch = D / CH;
  for (int e = wid; e < n; e += nw) {
    const S* wr = W + (long)e * D;
    float acc = 0.f;
    if (vec) {                                  // 16-byte loads of the router row, 4 in flight
      for (int c0 = lane; c0 < nch; c0 += 256) {
        uint4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          v[u] = c0 + u * 64 < nch ? *reinterpret_cast<const uint4*>(wr + (long)(c0 + u * 64) * CH)
                                   : uint4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (c0 + u * 64 >= nch) continue;
          const float* rr = row + (c0 + u * 64) * CH;
          if constexpr (sizeof(S) == 2) {
            float f[8];
            unpack8bf(v[u], f);
#pragma unroll
            for (int q = 0; q < 8; ++q) acc += rr[q] * f[q];
          } else {
            acc += rr[0] * __uint_as_float(v[u].x) + rr[1] * __uint_as_float(v[u].y) +
                   rr[2] * __uint_as_float(v[u].z) + rr[3] * __uint_as_float(v[u].w);
          }
        }
      }
    } else {
      for (int c = lane; c < D; c += 64) acc += row[c] * ldf(wr + c);
    }
    acc = wave_sum(acc);
    if (lane == 0) z[e] = acc + (bias != nullptr ? bias[e] : 0.f);
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  float m = -INFINITY;
  float sum = 0.f;
  float* wt = topk_w + (long)t * top;
  int* id = topk_ids + (long)t * top;
  for (int j = 0; j < top; ++j) {
    int best = -1;
    float bz = -INFINITY;
    for (int e = 0; e < n; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken |= id[i] == e;
      if (taken) continue;
      if (best < 0 || z[e] > bz) { best = e; bz = z[e]; }
    }
    id[j] = best;
    if (j == 0) m = bz;                          // the first pick is the largest logit
    const float ev = expf(bz - m);
    wt[j] = ev;
    sum += ev;
  }
  const float inv = 1.f / sum;
  for (int j = 0; j < top; ++j) wt[j] *= inv;
}

}  // namespace

#define DT_SWITCH(dt, CALL_BF16, CALL_F32) \
  do {                                     \
    if ((dt) == 0) { CALL_BF16; }          \
    else if ((dt) == 1) { CALL_F32; }      \
    else return (int)hipErrorInvalidValue; \
  } while (0)

extern "C" int dli_prev_tokens(int* prev, const int* ids, int* state, const int* slots,
                               const int* cu, const int* positions, int num_seqs, int max_seqlen,
                               hipStream_t st) {
  if (num_seqs <= 0 || max_seqlen <= 0) return 0;
  if (state == nullptr || slots == nullptr) return (int)hipErrorInvalidValue;
  prev_tokens_kernel<<<num_seqs, max_seqlen >= 256 ? 256 : 64, 0, st>>>(prev, ids, state, slots, cu,
                                                                       positions);
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_embedding_bigram(float* x, void* xs, const int* ids, const int* prev,
                                    const void* table, const void* bigram, int T, int dim,
                                    int vocab, int buckets, int mul_prev, int mul_cur, int dt,
                                    hipStream_t st) {
  if (T <= 0) return 0;
  if (bigram != nullptr && (prev == nullptr || buckets < 1)) return (int)hipErrorInvalidValue;
  const int nb = (int)(((long)T * dim + 255) / 256);
  DT_SWITCH(dt,
            (embedding_bigram_kernel<u16><<<nb, 256, 0, st>>>(
                x, (u16*)xs, ids, prev, (const u16*)table, (const u16*)bigram, T, dim, vocab,
                buckets, (long)mul_prev, (long)mul_cur)),
            (embedding_bigram_kernel<float><<<nb, 256, 0, st>>>(
                x, (float*)xs, ids, prev, (const float*)table, (const float*)bigram, T, dim,
                vocab, buckets, (long)mul_prev, (long)mul_cur)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_postnorm(float* x, const float* y, int ldy, float keep, const void* w,
                            const void* b, void* h, int rows, int dim, float eps,
                            const long* rows_idx, int dt, hipStream_t st) {
  if (rows <= 0) return 0;
  const size_t sh = (size_t)(dim + 16) * 4;
  if (dim < 1 || sh > 60000 || w == nullptr || b == nullptr || h == nullptr)
    return (int)hipErrorInvalidValue;
  const bool vec4 = dim % 4 == 0 && ldy % 4 == 0 &&
                    (((uintptr_t)x | (uintptr_t)y | (uintptr_t)w | (uintptr_t)b | (uintptr_t)h) & 15) == 0;
  DT_SWITCH(dt,
            (postnorm_kernel<u16><<<rows, 256, sh, st>>>(x, y, ldy, keep, (const u16*)w,
                                                         (const u16*)b, (u16*)h, dim, eps,
                                                         rows_idx, vec4)),
            (postnorm_kernel<float><<<rows, 256, sh, st>>>(x, y, ldy, keep, (const float*)w,
                                                           (const float*)b, (float*)h, dim, eps,
                                                           rows_idx, vec4)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_add_rmsnormed(float* x, const float* y, int ldy, const void* w, void* h,
                                 int rows, int dim, float eps, int dt, hipStream_t st) {
  if (rows <= 0) return 0;
  if (dim < 1) return (int)hipErrorInvalidValue;
  const bool vec4 = dim % 4 == 0 && ldy % 4 == 0 &&
                    (((uintptr_t)x | (uintptr_t)y | (uintptr_t)w | (uintptr_t)h) & 15) == 0;
  DT_SWITCH(dt,
            (add_rmsnormed_kernel<u16><<<rows, 256, 0, st>>>(x, y, ldy, (const u16*)w, (u16*)h,
                                                             dim, eps, vec4)),
            (add_rmsnormed_kernel<float><<<rows, 256, 0, st>>>(x, y, ldy, (const float*)w,
                                                               (float*)h, dim, eps, vec4)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_side_gate(void* out, const float* gate, int ldg, const int* ids,
                             const void* table, int ldt, int col0, int T, int n, int vocab,
                             int dt, hipStream_t st) {
  if (T <= 0 || n <= 0) return 0;
  if (col0 < 0 || col0 + n > ldt) return (int)hipErrorInvalidValue;
  const int nb = (int)(((long)T * n + 255) / 256);
  DT_SWITCH(dt,
            (side_gate_kernel<u16><<<nb, 256, 0, st>>>((u16*)out, gate, ldg, ids,
                                                       (const u16*)table, ldt, col0, T, n, vocab)),
            (side_gate_kernel<float><<<nb, 256, 0, st>>>((float*)out, gate, ldg, ids,
                                                         (const float*)table, ldt, col0, T, n,
                                                         vocab)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_rmsnorm_cols(void* out, const float* src, int lds, const void* w, int T, int n,
                                float eps, const float* gate, int ldg, int groups, int ldo,
                                float out_scale, int dt, hipStream_t st) {
  if (T <= 0) return 0;
  if (n < 1 || groups < 1) return (int)hipErrorInvalidValue;
  if ((long)T * groups <= 512 && n >= 1024) {
    DT_SWITCH(dt,
              (rmsnorm_cols_block_kernel<u16><<<T * groups, 256, 0, st>>>(
                  (u16*)out, src, lds, (const u16*)w, n, eps, gate, ldg, groups, ldo, out_scale)),
              (rmsnorm_cols_block_kernel<float><<<T * groups, 256, 0, st>>>(
                  (float*)out, src, lds, (const float*)w, n, eps, gate, ldg, groups, ldo,
                  out_scale)));
    DLI_RETURN_LAUNCH();
  }
  const int nb = (int)(((long)T * groups + 3) / 4);
  const bool vec4 = n % 4 == 0 && lds % 4 == 0 && ldg % 4 == 0 && ldo % 4 == 0 &&
                    (((uintptr_t)out | (uintptr_t)src | (uintptr_t)w | (uintptr_t)gate) & 15) == 0;
  DT_SWITCH(dt,
            (rmsnorm_cols_kernel<u16><<<nb, 256, 0, st>>>((u16*)out, src, lds, (const u16*)w, T,
                                                          n, eps, vec4, gate, ldg, groups, ldo,
                                                          out_scale)),
            (rmsnorm_cols_kernel<float><<<nb, 256, 0, st>>>((float*)out, src, lds,
                                                            (const float*)w, T, n, eps, vec4,
                                                            gate, ldg, groups, ldo, out_scale)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_latent_prepare(const float* qproj, int ldq, const float* kvproj, int ldkv,
                                  const void* cw, float eps, int T, int H, int d, int dr, int r,
                                  int rot_dims, const double* inv_freq, const int* positions,
                                  const int* slots, void* q_nope, void* q_full, void* cache,
                                  int half, int dt, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot_dims > dr || (rot_dims & 1) || rot_dims > 8192 || H < 1 || d < 1 || r < 1)
    return (int)hipErrorInvalidValue;
  if (kvproj != nullptr && (cw == nullptr || cache == nullptr || slots == nullptr))
    return (int)hipErrorInvalidValue;
  DT_SWITCH(dt,
            (latent_prepare_kernel<u16><<<T, 256, (size_t)rot_dims * 4, st>>>(
                qproj, ldq, kvproj, ldkv, (const u16*)cw, eps, H, d, dr, r, rot_dims, inv_freq,
                positions, slots, (u16*)q_nope, (u16*)q_full, (u16*)cache, half != 0)),
            (latent_prepare_kernel<float><<<T, 256, (size_t)rot_dims * 4, st>>>(
                qproj, ldq, kvproj, ldkv, (const float*)cw, eps, H, d, dr, r, rot_dims, inv_freq,
                positions, slots, (float*)q_nope, (float*)q_full, (float*)cache, half != 0)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_head_gate(void* out, const float* o, const float* g, int ldg, int T, int H,
                             int n, int dt, hipStream_t st) {
  if (T <= 0) return 0;
  const int nb = (int)(((long)T * H * n + 255) / 256);
  DT_SWITCH(dt, (head_gate_kernel<u16><<<nb, 256, 0, st>>>((u16*)out, o, g, ldg, T, H, n)),
            (head_gate_kernel<float><<<nb, 256, 0, st>>>((float*)out, o, g, ldg, T, H, n)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_logit_router(float* topk_w, int* topk_ids, const void* h, int ldh,
                                const void* W, const float* bias, int T, int D, int n, int top,
                                int dt, hipStream_t st) {
  if (T <= 0) return 0;
  if (n < 1 || top < 1 || top > n || n > ROUTER_MAX || (size_t)(D + n) * 4 > 60000)
    return (int)hipErrorInvalidValue;
  const size_t sh = (size_t)(D + n) * 4;
  const bool vec = (uintptr_t)W % 16 == 0 && D % (dt == 0 ? 8 : 4) == 0;
  DT_SWITCH(dt,
            (logit_router_kernel<u16><<<T, 256, sh, st>>>(topk_w, topk_ids, (const u16*)h, ldh,
                                                          (const u16*)W, bias, D, n, top, vec)),
            (logit_router_kernel<float><<<T, 256, sh, st>>>(topk_w, topk_ids, (const float*)h,
                                                            ldh, (const float*)W, bias, D, n,
                                                            top, vec)));
  DLI_RETURN_LAUNCH();
}
