// Row kernels of the hybrid (mixed attention / recurrent) model family, whose residual stream
// and norms are fp32 while the GEMM operands keep the model's storage type.
//
// Every kernel is built for two storage types: bf16 (dt = 0, the serving format) and fp32
// (dt = 1, the exact mode, where weights, GEMM operands and caches are all fp32). "S" below is
// that storage type; residuals, projection outputs that feed a norm, a gate or a recurrence,
// and all arithmetic are fp32 in both.
//
//  * embedding_f32      x[t] = table[ids[t]] * scale (+ pos_table[positions[t]]) as fp32 (two
//                       copies: the stream and the loop input)
//  * resadd_groupnorm   x = keep * x + mult * y + bias; h = grouped RMS norm of x * gain (S out,
//                       or unrounded fp32 for a consumer that mixes rows first)
//  * token_shift        u[t] = h[t] + (h[t-1] - h[t]) * mu over the normed fp32 rows, h[t-1] of a
//                       portion's first row from the sequence's state slot
//  * talk_prepare       q / k / v bias, unit-RMS q and k heads, k and v -> cache, queries with
//                       the pre-softmax head mixing folded in -> S
//  * concat_cast        [x ; x0] fp32 -> S rows of width 2D (the operand of the loop-entry GEMM)
//  * act_mul            gelu_tanh(gate) * up, silu(gate) * up, gelu_tanh(up), gelu_erf(up) or a
//                       plain copy over a fp32 projection -> S [T, F]
//  * attn_prepare       per-head RMS norm of q and k (shared weights), normed k -> key cache,
//                       raw k -> value cache ("values are the keys"), normed q -> S
//  * mla_prepare        latent attention: RMS norm of the compressed kv -> cache, interleaved
//                       rotary on the shared rotated key -> cache, rotary on each head's rotated
//                       query part; the unrotated query parts go to a GEMM operand
#include "common.h"

namespace {

template <typename S> __device__ __forceinline__ float ldf(const S* p);
template <> __device__ __forceinline__ float ldf<u16>(const u16* p) { return bf2f(*p); }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename S> __device__ __forceinline__ void stf(S* p, float v);
template <> __device__ __forceinline__ void stf<u16>(u16* p, float v) { *p = f2bf(v); }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

template <typename S>
__global__ void __launch_bounds__(256) embedding_f32_kernel(
    float* __restrict__ x, float* __restrict__ x0, const int* __restrict__ ids,
    const S* __restrict__ table, int T, int dim, int vocab, float scale,
    const S* __restrict__ pos_table, const int* __restrict__ positions, int max_pos) {
  const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long)T * dim) return;
  const int t = (int)(gid / dim), c = (int)(gid % dim);
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  float v = ldf(table + (long)id * dim + c) * scale;
  if (pos_table != nullptr) {
    int p = positions[t];
    p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
    v += ldf(pos_table + (long)p * dim + c);
  }
  x[gid] = v;
  if (x0 != nullptr) x0[gid] = v;
}

// One workgroup per row. x (fp32, in place): x = keep * x + mult * y + bias, y and bias may be
// null. The row is cut into `groups` equal parts, each scaled by its own rsqrt(mean(sq) + eps);
// h = that * w. h may be null (the last layer's add). rows_idx (nullable) selects source rows
// (the final norm of the rows whose logits are wanted); it excludes y / bias / the write-back.
template <typename S>
__global__ void __launch_bounds__(256) resadd_groupnorm_kernel(
    float* __restrict__ x, const float* __restrict__ y, int ldy, const S* __restrict__ bias,
    float keep, float mult, const S* __restrict__ w, void* __restrict__ h, int ldh, int dim,
    int groups, float eps, const long* __restrict__ rows_idx, bool vec4, float gain,
    bool h_f32, float w_offset) {
  extern __shared__ __attribute__((aligned(16))) float row[];   // dim floats + group scales
  float* gsum = row + dim;
  const int r = blockIdx.x;
  const long src = rows_idx ? rows_idx[r] : r;
  float* xr = x + src * dim;
  for (int g = threadIdx.x; g < groups; g += blockDim.x) gsum[g] = 0.f;
  const bool update = rows_idx == nullptr && (y != nullptr || bias != nullptr || keep != 1.f);
  if (vec4) {                               // 16-byte loads and stores of the fp32 rows
    for (int c = threadIdx.x * 4; c < dim; c += blockDim.x * 4) {
      f32x4 v = *reinterpret_cast<const f32x4*>(xr + c);
      if (rows_idx == nullptr) {
        if (keep == 0.f) v = f32x4{0.f, 0.f, 0.f, 0.f};
        else if (keep != 1.f) v *= keep;
        if (y != nullptr) v += mult * *reinterpret_cast<const f32x4*>(y + (long)r * ldy + c);
        if (bias != nullptr) {
#pragma unroll
          for (int u = 0; u < 4; ++u) v[u] += ldf(bias + c + u);
        }
        if (update) *reinterpret_cast<f32x4*>(xr + c) = v;
      }
      *reinterpret_cast<f32x4*>(row + c) = v;
    }
  } else {
    for (int c = threadIdx.x; c < dim; c += blockDim.x) {
      float v = xr[c];
      if (rows_idx == nullptr) {
        v = keep != 0.f ? v * keep : 0.f;
        if (y != nullptr) v += mult * y[(long)r * ldy + c];
        if (bias != nullptr) v += ldf(bias + c);
        if (update) xr[c] = v;
      }
      row[c] = v;
    }
  }
  __syncthreads();
  if (h == nullptr) return;
  const int gl = dim / groups;
  // one wave per group, in turn: a wave sums its group's squares in a fixed order
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int g = wid; g < groups; g += nw) {
    float s = 0.f;
    for (int c = lane; c < gl; c += 64) { const float v = row[g * gl + c]; s += v * v; }
    s = wave_sum(s);
    if (lane == 0) gsum[g] = 1.f / sqrtf(s / (float)gl + eps);
  }
  __syncthreads();
  if (h_f32) {
    for (int c = threadIdx.x; c < dim; c += blockDim.x)
      ((float*)h)[(long)r * ldh + c] = row[c] * gsum[c / gl] * (ldf(w + c) + w_offset) * gain;
  } else {
    for (int c = threadIdx.x; c < dim; c += blockDim.x)
      stf((S*)h + (long)r * ldh + c, row[c] * gsum[c / gl] * (ldf(w + c) + w_offset) * gain);
  }
}

// Token shift over normed fp32 rows: u[t] = h[t] + (h[t-1] - h[t]) * mu. Grid (row blocks of a
// sequence, sequences, column blocks). h[t-1] of a portion's first row is the sequence's row
// of `state` (zeros at position 0). The workgroup that holds a portion's first row also stores
// the portion's LAST row into the state, after it has read the old one: every thread reads and
// then writes the same columns, so the order holds without a second launch. Sequences
// without a slot (padding rows of a captured step) pass through unshifted. VEC = 4: 16-byte
// loads of the fp32 rows (dim a multiple of 4).
constexpr int SHIFT_ROWS = 4;
template <typename S, int VEC>
__global__ void __launch_bounds__(256) token_shift_kernel(
    const float* __restrict__ h, const S* __restrict__ mu, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ cu, const int* __restrict__ positions,
    S* __restrict__ out, int dim) {
  const int s = blockIdx.y;
  const int t0 = cu[s], t1 = cu[s + 1];
  const int r0 = blockIdx.x * SHIFT_ROWS;
  if (t0 + r0 >= t1) return;
  const int slot = slots != nullptr ? slots[s] : -1;
  const int rows = min(SHIFT_ROWS, t1 - t0 - r0);
  const bool from_zero = positions[t0] == 0;
  const int c = (blockIdx.z * blockDim.x + threadIdx.x) * VEC;
  if (c >= dim) return;
  float m[VEC], prev[VEC], cur[VEC];
#pragma unroll
  for (int u = 0; u < VEC; ++u) { m[u] = ldf(mu + c + u); prev[u] = 0.f; }
  auto load = [&](const float* p, float* v) {
    if constexpr (VEC == 4) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(p);
      v[0] = q[0]; v[1] = q[1]; v[2] = q[2]; v[3] = q[3];
    } else {
      v[0] = *p;
    }
  };
  if (r0 > 0) load(h + (long)(t0 + r0 - 1) * dim + c, prev);
  else if (slot >= 0 && !from_zero) load(state + (long)slot * dim + c, prev);
  for (int i = 0; i < rows; ++i) {
    const long o = (long)(t0 + r0 + i) * dim + c;
    load(h + o, cur);
#pragma unroll
    for (int u = 0; u < VEC; ++u) {
      stf(out + o + u, slot < 0 ? cur[u] : cur[u] + (prev[u] - cur[u]) * m[u]);
      prev[u] = cur[u];
    }
  }
  if (r0 == 0 && slot >= 0) {
    load(h + (long)(t1 - 1) * dim + c, cur);
#pragma unroll
    for (int u = 0; u < VEC; ++u) state[(long)slot * dim + c + u] = cur[u];
  }
}

template <typename S>
__global__ void __launch_bounds__(256) concat_cast_kernel(
    S* __restrict__ out, const float* __restrict__ a, const float* __restrict__ b, int T,
    int dim) {
  const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long)T * 2 * dim) return;
  const int t = (int)(gid / (2 * dim)), c = (int)(gid % (2 * dim));
  stf(out + gid, c < dim ? a[(long)t * dim + c] : b[(long)t * dim + c - dim]);
}

__device__ __forceinline__ float gelu_tanh32(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

__device__ __forceinline__ float act_pair(int kind, float g, float u, float limit) {
  if (kind == 5) {                       // clamped swish: min / clamp, then g sigmoid(1.702 g) (u + 1)
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.f + expf(-1.702f * g)) * (u + 1.f);
  }
  if (kind == 0) return gelu_tanh32(g) * u;
  if (kind == 1) return g / (1.f + expf(-g)) * u;
  if (kind == 3) return 0.5f * g * (1.f + erff(g * 0.7071067811865476f));
  if (kind == 4) return g;
  return gelu_tanh32(g);
}

// kind 0: gelu_tanh(gu[:, c]) * gu[:, F + c]; 1: silu(..) * ..; 2: gelu_tanh(gu[:, c]);
// 3: the exact (erf) GELU of gu[:, c]; 4: gu[:, c] itself (a rounding copy of a column slice);
// 5: g sigmoid(1.702 g) (u + 1) with g = min(gu[:, c], limit), u = clamp(gu[:, F + c], +-limit).
// nrows (nullable, device): rows from *nrows on hold no data and are skipped.
// I: the projection's type (fp32, or bf16 bits when a tuned GEMM wrote it).
template <typename I> __device__ __forceinline__ f32x4 ldin4(const I* p);
template <> __device__ __forceinline__ f32x4 ldin4<float>(const float* p) {
  return *reinterpret_cast<const f32x4*>(p);
}
template <> __device__ __forceinline__ f32x4 ldin4<u16>(const u16* p) {
  const uint2 b = *reinterpret_cast<const uint2*>(p);
  return f32x4{__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xffff0000u),
               __uint_as_float(b.y << 16), __uint_as_float(b.y & 0xffff0000u)};
}

template <typename S, typename I>
__global__ void __launch_bounds__(256) act_mul_kernel(
    S* __restrict__ out, int ldo, const I* __restrict__ gu, int ldg, int T, int F, int kind,
    const int* __restrict__ nrows, float limit) {
  const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (long)T * F) return;
  const int t = (int)(gid / F), c = (int)(gid % F);
  if (nrows != nullptr && t >= *nrows) return;
  const I* r = gu + (long)t * ldg;
  stf(out + (long)t * ldo + c,
      act_pair(kind, ldf(r + c), (kind >= 2 && kind != 5) ? 0.f : ldf(r + F + c), limit));
}

// 4 features a thread (F, ldg multiples of 4, 16-byte aligned rows): 16-byte loads
template <typename S, typename I>
__global__ void __launch_bounds__(256) act_mul4_kernel(
    S* __restrict__ out, int ldo, const I* __restrict__ gu, int ldg, int T, int F, int kind,
    const int* __restrict__ nrows, float limit) {
  const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int f4 = F >> 2;
  if (gid >= (long)T * f4) return;
  const int t = (int)(gid / f4), c = (int)(gid % f4) * 4;
  if (nrows != nullptr && t >= *nrows) return;
  const I* r = gu + (long)t * ldg;
  const f32x4 g = ldin4(r + c);
  f32x4 u = f32x4{0.f, 0.f, 0.f, 0.f};
  if (kind < 2 || kind == 5) u = ldin4(r + F + c);
#pragma unroll
  for (int i = 0; i < 4; ++i)
    stf(out + (long)t * ldo + c + i, act_pair(kind, g[i], u[i], limit));
}

// Grid (token, head slices). proj row (fp32, + bias): [H*d q | G*d k | G*dv v] (q only when the
// layer attends another layer's cache: kcache null). q and k heads are divided by their RMS;
// k and v go to the cache row (by slice 0); the queries leave with the pre-softmax head mixing
// folded in:
//   sum_g talk[h][g] (q_g . k_c(g)) = sum_c (sum_{g in c} talk[h][g] q_g) . k_c
// so head h carries q'_h [G*d] whose part c is sum_{g in c} talk[h][g] q_g, and scores whole
// cached key rows. Every slice norms all query heads (cheap) and writes the mixed queries of
// its own heads [h0, h1), VEC consecutive columns a thread.
template <typename S, int VEC>
__global__ void __launch_bounds__(256) talk_prepare_kernel(
    const float* __restrict__ proj, int ldp, const S* __restrict__ bias,
    const float* __restrict__ talk, float eps, int H, int G, int d, int dv,
    S* __restrict__ q_out, S* __restrict__ kcache, S* __restrict__ vcache,
    const int* __restrict__ slots) {
  extern __shared__ __attribute__((aligned(16))) float qn[];   // [H * d] unit-RMS queries, [H * H] talk
  float* tk = qn + H * d;
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const float* row = proj + (long)t * ldp;
  const int slot = (kcache != nullptr && blockIdx.y == 0) ? slots[t] : -1;
  const int units = H + (slot >= 0 ? G : 0);
  for (int i = threadIdx.x; i < H * H; i += blockDim.x) tk[i] = talk[i];
  for (int u = wid; u < units; u += nw) {
    const int off = u * d;                            // q heads, then k heads, are contiguous
    float ss = 0.f;
    for (int c = lane; c < d; c += 64) { const float v = row[off + c] + ldf(bias + off + c); ss += v * v; }
    ss = wave_sum(ss);
    const float rs = 1.f / sqrtf(ss / (float)d + eps);
    if (u < H) {
      for (int c = lane; c < d; c += 64) qn[off + c] = (row[off + c] + ldf(bias + off + c)) * rs;
    } else {
      S* kd = kcache + ((long)slot * G + (u - H)) * d;
      for (int c = lane; c < d; c += 64) stf(kd + c, (row[off + c] + ldf(bias + off + c)) * rs);
    }
  }
  if (slot >= 0) {
    const int voff = (H + G) * d;
    S* vd = vcache + (long)slot * G * dv;
    for (int c = threadIdx.x; c < G * dv; c += blockDim.x)
      stf(vd + c, row[voff + c] + ldf(bias + voff + c));
  }
  __syncthreads();
  const int rep = H / G, wq = G * d;
  const int per = (H + gridDim.y - 1) / gridDim.y;
  const int h0 = blockIdx.y * per, h1 = min(H, h0 + per);
  S* qo = q_out + (long)t * H * wq;
  for (int i = h0 * wq + threadIdx.x * VEC; i < h1 * wq; i += blockDim.x * VEC) {
    const int h = i / wq, rem = i % wq, c = rem / d, col = rem % d;   // VEC | d: one (h, c)
    const float* tr = tk + h * H + c * rep;
    const float* qs = qn + (c * rep) * d + col;
    float acc[VEC];
#pragma unroll
    for (int u = 0; u < VEC; ++u) acc[u] = 0.f;
    for (int r = 0; r < rep; ++r) {
      const float w = tr[r];
#pragma unroll
      for (int u = 0; u < VEC; ++u) acc[u] += w * qs[r * d + u];
    }
    if constexpr (VEC == 8 && sizeof(S) == 2) {
      store8((u16*)qo + i, acc);
    } else {
#pragma unroll
      for (int u = 0; u < VEC; ++u) stf(qo + i + u, acc[u]);
    }
  }
}

// proj row: [H*d q | G*d k | ...]; one wave per (token, head) unit, H + G units per token.
template <typename S>
__global__ void __launch_bounds__(256) attn_prepare_kernel(
    const float* __restrict__ proj, int ldp, const S* __restrict__ qw, const S* __restrict__ kw,
    float eps, int T, int H, int G, int d, S* __restrict__ q_out, S* __restrict__ kcache,
    S* __restrict__ vcache, const int* __restrict__ slots) {
  const int lane = threadIdx.x & 63;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= (long)T * (H + G)) return;
  const int t = (int)(unit / (H + G)), u = (int)(unit % (H + G));
  const bool is_q = u < H;
  const float* src = proj + (long)t * ldp + (is_q ? u * d : H * d + (u - H) * d);
  float s = 0.f;
  for (int c = lane; c < d; c += 64) { const float v = src[c]; s += v * v; }
  s = wave_sum(s);
  const float rs = 1.f / sqrtf(s / (float)d + eps);
  if (is_q) {
    S* dst = q_out + ((long)t * H + u) * d;
    for (int c = lane; c < d; c += 64) stf(dst + c, src[c] * rs * ldf(qw + c));
  } else {
    const int slot = slots[t];
    if (slot < 0) return;
    const int g = u - H;
    S* kd = kcache + ((long)slot * G + g) * d;
    S* vd = vcache + ((long)slot * G + g) * d;
    for (int c = lane; c < d; c += 64) {
      const float v = src[c];
      stf(kd + c, v * rs * ldf(kw + c));
      stf(vd + c, v);
    }
  }
}

// proj row: [H*(d+dr) q | r compressed kv | dr shared rotated key]. One workgroup per token.
//  cache row (width r + dr): [normed latent | rotated key]
//  q_nope [T, H, d] (S): operand of the per-head absorb GEMM
//  q_full [T, H, r + dr] (S): this kernel writes the rotated tail [r, r+dr) of every head
// inv_freq [rot_dims / 2] fp64; pairs (2i, 2i+1) of the first rot_dims of the dr part rotate.
template <typename S>
__global__ void __launch_bounds__(256) mla_prepare_kernel(
    const float* __restrict__ proj, int ldp, const S* __restrict__ cw, float eps, int T, int H,
    int d, int dr, int r, int rot_dims, const double* __restrict__ inv_freq,
    const int* __restrict__ positions, const int* __restrict__ slots, S* __restrict__ q_nope,
    S* __restrict__ q_full, S* __restrict__ cache) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const float* row = proj + (long)t * ldp;
  const float* dkv = row + (long)H * (d + dr);
  const double pos = (double)positions[t];
  const int slot = slots[t];
  float s = 0.f;
  for (int c = threadIdx.x; c < r; c += blockDim.x) { const float v = dkv[c]; s += v * v; }
  s = block_sum(s, red);
  const float rs = 1.f / sqrtf(s / (float)r + eps);
  if (slot >= 0) {
    S* cr = cache + (long)slot * (r + dr);
    for (int c = threadIdx.x; c < r; c += blockDim.x) stf(cr + c, dkv[c] * rs * ldf(cw + c));
    for (int c = threadIdx.x; c < dr; c += blockDim.x) {
      float v = dkv[r + c];
      if (c < rot_dims) {
        const double a = pos * inv_freq[c >> 1];   // the angle in double, rounded once
        const float cs = (float)cos(a), sn = (float)sin(a);
        const float o = dkv[r + (c ^ 1)];
        v = (c & 1) ? v * cs + o * sn : v * cs - o * sn;
      }
      stf(cr + r + c, v);
    }
  }
  for (int i = threadIdx.x; i < H * (d + dr); i += blockDim.x) {
    const int h = i / (d + dr), c = i % (d + dr);
    float v = row[i];
    if (c < d) {
      stf(q_nope + ((long)t * H + h) * d + c, v);
    } else {
      const int cc = c - d;
      if (cc < rot_dims) {
        const double a = pos * inv_freq[cc >> 1];
        const float cs = (float)cos(a), sn = (float)sin(a);
        const float o = row[h * (d + dr) + d + (cc ^ 1)];
        v = (cc & 1) ? v * cs + o * sn : v * cs - o * sn;
      }
      stf(q_full + ((long)t * H + h) * (r + dr) + r + cc, v);
    }
  }
}

}  // namespace

#define DT_SWITCH(dt, CALL_BF16, CALL_F32) \
  do {                                     \
    if ((dt) == 0) { CALL_BF16; }          \
    else if ((dt) == 1) { CALL_F32; }      \
    else return (int)hipErrorInvalidValue; \
  } while (0)

extern "C" int dli_embedding_f32(float* x, float* x0, const int* ids, const void* table, int T,
                                 int dim, int vocab, float scale, const void* pos_table,
                                 const int* positions, int max_pos, int dt, hipStream_t st) {
  if (T <= 0) return 0;
  if (pos_table != nullptr && (positions == nullptr || max_pos < 1))
    return (int)hipErrorInvalidValue;
  const int nb = (int)(((long)T * dim + 255) / 256);
  DT_SWITCH(dt,
            (embedding_f32_kernel<u16><<<nb, 256, 0, st>>>(x, x0, ids, (const u16*)table, T, dim,
                                                          vocab, scale, (const u16*)pos_table,
                                                          positions, max_pos)),
            (embedding_f32_kernel<float><<<nb, 256, 0, st>>>(x, x0, ids, (const float*)table, T,
                                                            dim, vocab, scale,
                                                            (const float*)pos_table, positions,
                                                            max_pos)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_resadd_groupnorm(float* x, const float* y, int ldy, const void* bias,
                                    float keep, float mult, const void* w, void* h, int ldh,
                                    int rows, int dim, int groups, float eps,
                                    const long* rows_idx, float gain, int h_f32, float w_offset,
                                    int dt, hipStream_t st) {
  if (rows <= 0) return 0;
  if (groups < 1 || dim % groups || (size_t)(dim + groups) * 4 > 60000)
    return (int)hipErrorInvalidValue;
  const size_t sh = (size_t)(dim + groups) * 4;
  const bool vec4 = dim % 4 == 0 && (uintptr_t)x % 16 == 0 &&
                    (y == nullptr || ((uintptr_t)y % 16 == 0 && ldy % 4 == 0));
  DT_SWITCH(dt,
            (resadd_groupnorm_kernel<u16><<<rows, 256, sh, st>>>(
                x, y, ldy, (const u16*)bias, keep, mult, (const u16*)w, h, ldh, dim, groups,
                eps, rows_idx, vec4, gain, h_f32 != 0, w_offset)),
            (resadd_groupnorm_kernel<float><<<rows, 256, sh, st>>>(
                x, y, ldy, (const float*)bias, keep, mult, (const float*)w, h, ldh, dim,
                groups, eps, rows_idx, vec4, gain, h_f32 != 0, w_offset)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_concat_cast(void* out, const float* a, const float* b, int T, int dim, int dt,
                               hipStream_t st) {
  if (T <= 0) return 0;
  const int nb = (int)(((long)T * 2 * dim + 255) / 256);
  DT_SWITCH(dt, (concat_cast_kernel<u16><<<nb, 256, 0, st>>>((u16*)out, a, b, T, dim)),
            (concat_cast_kernel<float><<<nb, 256, 0, st>>>((float*)out, a, b, T, dim)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_token_shift(const float* h, const void* mu, float* state, const int* slots,
                               const int* cu, const int* positions, void* out, int num_seqs,
                               int max_seqlen, int dim, int dt, hipStream_t st) {
  if (num_seqs <= 0 || max_seqlen <= 0) return 0;
  if (num_seqs > 65535) return (int)hipErrorInvalidValue;
  const bool v4 = dim % 4 == 0 && (uintptr_t)h % 16 == 0 && (uintptr_t)state % 16 == 0;
  const int per = 256 * (v4 ? 4 : 1);
  dim3 grid((max_seqlen + SHIFT_ROWS - 1) / SHIFT_ROWS, num_seqs, (dim + per - 1) / per);
#define SHIFT_LAUNCH(S, V)                                                                    \
  token_shift_kernel<S, V><<<grid, 256, 0, st>>>(h, (const S*)mu, state, slots, cu, positions, \
                                                 (S*)out, dim)
  if (v4) DT_SWITCH(dt, (SHIFT_LAUNCH(u16, 4)), (SHIFT_LAUNCH(float, 4)));
  else DT_SWITCH(dt, (SHIFT_LAUNCH(u16, 1)), (SHIFT_LAUNCH(float, 1)));
#undef SHIFT_LAUNCH
  DLI_RETURN_LAUNCH();
}

// in_dt: type of the projection gu (1 fp32; 0 bf16, with bf16 output only)
extern "C" int dli_act_mul(void* out, int ldo, const void* gu, int ldg, int T, int F, int kind,
                           const int* nrows, float limit, int in_dt, int dt, hipStream_t st) {
  if (T <= 0) return 0;
  if (kind < 0 || kind > 5 || in_dt < 0 || in_dt > 1 || (in_dt == 0 && dt != 0))
    return (int)hipErrorInvalidValue;
  const bool v4 = F % 4 == 0 && ldg % 4 == 0 && (uintptr_t)gu % 16 == 0;
  const int nb = (int)(((long)T * (v4 ? F / 4 : F) + 255) / 256);
  if (in_dt == 0) {
    if (v4) act_mul4_kernel<u16, u16><<<nb, 256, 0, st>>>((u16*)out, ldo, (const u16*)gu, ldg, T, F, kind, nrows, limit);
    else act_mul_kernel<u16, u16><<<nb, 256, 0, st>>>((u16*)out, ldo, (const u16*)gu, ldg, T, F, kind, nrows, limit);
    DLI_RETURN_LAUNCH();
  }
  const float* gf = (const float*)gu;
  if (v4)
    DT_SWITCH(dt,
              (act_mul4_kernel<u16, float><<<nb, 256, 0, st>>>((u16*)out, ldo, gf, ldg, T, F, kind, nrows, limit)),
              (act_mul4_kernel<float, float><<<nb, 256, 0, st>>>((float*)out, ldo, gf, ldg, T, F, kind, nrows, limit)));
  else
    DT_SWITCH(dt, (act_mul_kernel<u16, float><<<nb, 256, 0, st>>>((u16*)out, ldo, gf, ldg, T, F, kind, nrows, limit)),
              (act_mul_kernel<float, float><<<nb, 256, 0, st>>>((float*)out, ldo, gf, ldg, T, F, kind, nrows, limit)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_talk_prepare(const float* proj, int ldp, const void* bias, const float* talk,
                                float eps, int T, int H, int G, int d, int dv, void* q_out,
                                void* kcache, void* vcache, const int* slots, int dt,
                                hipStream_t st) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || H % G || d < 1 || dv < 1 || (kcache == nullptr) != (vcache == nullptr))
    return (int)hipErrorInvalidValue;
  const size_t sh = ((size_t)H * d + (size_t)H * H) * 4;
  if (sh > 60000) return (int)hipErrorInvalidValue;
  // few tokens (decode steps): the heads of a token are dealt to several workgroups
  int slices = 1;
  while (slices < H && slices < 16 && (long)T * slices < 1024) slices *= 2;
  if (slices > H) slices = H;
  dim3 grid(T, slices);
  const bool v8 = d % 8 == 0 && (uintptr_t)q_out % 16 == 0;
#define TALK_LAUNCH(S, V)                                                                   \
  talk_prepare_kernel<S, V><<<grid, 256, sh, st>>>(proj, ldp, (const S*)bias, talk, eps, H, G, \
                                                   d, dv, (S*)q_out, (S*)kcache, (S*)vcache, slots)
  if (v8) DT_SWITCH(dt, (TALK_LAUNCH(u16, 8)), (TALK_LAUNCH(float, 8)));
  else DT_SWITCH(dt, (TALK_LAUNCH(u16, 1)), (TALK_LAUNCH(float, 1)));
#undef TALK_LAUNCH
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_attn_prepare(const float* proj, int ldp, const void* qw, const void* kw,
                                float eps, int T, int H, int G, int d, void* q_out, void* kcache,
                                void* vcache, const int* slots, int dt, hipStream_t st) {
  if (T <= 0) return 0;
  const long units = (long)T * (H + G);
  const int nb = (int)((units + 3) / 4);
  DT_SWITCH(dt,
            (attn_prepare_kernel<u16><<<nb, 256, 0, st>>>(
                proj, ldp, (const u16*)qw, (const u16*)kw, eps, T, H, G, d, (u16*)q_out,
                (u16*)kcache, (u16*)vcache, slots)),
            (attn_prepare_kernel<float><<<nb, 256, 0, st>>>(
                proj, ldp, (const float*)qw, (const float*)kw, eps, T, H, G, d, (float*)q_out,
                (float*)kcache, (float*)vcache, slots)));
  DLI_RETURN_LAUNCH();
}

extern "C" int dli_mla_prepare(const float* proj, int ldp, const void* cw, float eps, int T,
                               int H, int d, int dr, int r, int rot_dims, const double* inv_freq,
                               const int* positions, const int* slots, void* q_nope,
                               void* q_full, void* cache, int dt, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot_dims > dr || (rot_dims & 1)) return (int)hipErrorInvalidValue;
  DT_SWITCH(dt,
            (mla_prepare_kernel<u16><<<T, 256, 0, st>>>(
                proj, ldp, (const u16*)cw, eps, T, H, d, dr, r, rot_dims, inv_freq, positions,
                slots, (u16*)q_nope, (u16*)q_full, (u16*)cache)),
            (mla_prepare_kernel<float><<<T, 256, 0, st>>>(
                proj, ldp, (const float*)cw, eps, T, H, d, dr, r, rot_dims, inv_freq, positions,
                slots, (float*)q_nope, (float*)q_full, (float*)cache)));
  DLI_RETURN_LAUNCH();
}
