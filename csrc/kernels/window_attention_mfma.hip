// MFMA form of the windowed attention of window_attention.hip (same arguments, same options,
// bf16 storage): one workgroup of 8 waves per (sequence, tile of 16 consecutive query tokens,
// 128-wide slice of the value dimension), all heads in the workgroup because the head-mixing
// matrix needs every head's normalised weights at the same (query, key).
//
// With head mixing, two passes over the window in tiles of 32 keys (without it an unsplit
// launch runs the usual single pass with rescaled accumulators):
//   pass 1   S^T = K . Q^T per head (v_mfma_f32_16x16x32_bf16, K rows as operand A, so a lane
//            holds 8 keys of ONE query: max / sum reduce over 2 shuffles), running max m and
//            sum l per (head, query) in registers.
//   pass 2   S^T again, w = exp(s - m) / l, stored bf16 as Pm[(query, key)][head]; the mix
//            W' = talk . W is an MFMA with talk as operand A and Pm rows as operand B; W'
//            lands as Pp[head][query][key]; then O += W' . V with W' rows as operand A and the
//            V tile, staged transposed (Vt[dim][key]), as operand B.
// With mixing, heads are dealt to waves round-robin (head h -> wave h % 8, at most 4 heads a
// wave, H <= 32, 128-wide value slices); without it, the wide form takes 8 heads a workgroup.
// Staging: the cache rows of the whole window are looked up once (slot table in LDS); a tile's
// K rows of every kv head that fits go to LDS by LDS-DMA (global_load_lds_dwordx4, padded rows,
// all pieces in flight); the V tile shares that LDS region (the two are never live together)
// and is transposed through registers. Query fragments come from global memory (L2), four at
// a time, the first group of a step requested together with the K tile: with 576-wide latent
// queries they fit neither registers nor the LDS left beside the weight tiles.
// Scores live in the log2 domain (scale and slope carry log2 e): one v_exp_f32 per weight.
//
// Masked positions (outside the window, after the query, past the sequence, rows past the
// tile's last query) get weight 0; a query row always sees itself, so l > 0.
#include "common.h"

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

namespace {

constexpr int TQ = 16, TK = 32, NW = 8, MAXHW = 4, MAXDVB = 8;
constexpr float LOG2E = 1.4426950408889634f;

struct MfmaArgs {
  const u16* q; int ldq;
  const u16* k; long k_stride;
  const u16* v; long v_stride;
  u16* out; int ldo;
  const float* gate; int ldg;
  const float* slopes;
  const float* talk;
  const int* cu; const int* positions;
  const int* block_tables; int bt_stride; int block_size;
  int H, G, dq, dv, window;
  float scale;
  // Gk: key heads per cache row (the values have G; Gk = 1: every head scores the whole key
  // row). chunk > 0: a query sees only keys of its own block of `chunk` positions.
  int Gk, chunk;
  int Hp;        // H rounded up to 32 (mix K dimension)
  int CG;        // kv heads staged per step
  // key-split form (few query tiles, long windows: decode steps): the window's tiles are dealt
  // to nsplit workgroups; mode 1 = pass 1 only (partial max / sum -> stats_ws), mode 2 = pass 2
  // only (the partials combined first; un-gated fp32 partial outputs -> o_ws), mode 0 = both
  int mode, nsplit, ndvs;
  // wide form (no head mixing, so heads need not share a workgroup): 8 heads a workgroup,
  // one per wave, and the wave's 32 accumulator blocks cover a 512-wide value slice instead
  // of 4 heads x 128 — latent attention's 512-wide values without recomputing the scores
  int wide, nhs;
  // rows-are-heads form of a decode step whose heads all share one cached row per position
  // (latent attention): the launcher presents token t's H heads as H query rows of a
  // one-head problem, all at token t's position: rowmul = H (cu and positions are per token)
  int rowmul;
  // rows-are-heads with grouped values (the key row is shared by all heads, the values are
  // not): vrows = heads per value group; row (= head) r applies its weights to group r / vrows
  int vrows;
  // value groups staged per apply step (they are packed at their own stride into the K regions)
  int cgv;
  // > 0: the cache rows of the whole window (slot_cap ints) are looked up once at kernel start
  // instead of per key tile (one global round trip and one barrier less per tile)
  int slot_cap;
  // sink != null (forms without head mixing): exp(sink[h]) joins head h's softmax denominator,
  // a key without a value counted once: the running (max, sum) of the first key split start
  // from (sink, 1) instead of (-inf, 0). head_gate: the gate row holds one number per head.
  // out_scale multiplies the output.
  const float* sink; int head_gate; float out_scale;
  // value slice of a workgroup: 128 with all heads in it; in the wide form the whole value
  // width up to 512 (narrower values take a narrower LDS image, so more workgroups share a CU)
  int dvw;
  float* stats_ws;   // [S][q tiles][nsplit][H][TQ][2]
  float* o_ws;       // [nsplit][T][H*dv]
  long o_ws_stride;  // T * H * dv
};

__device__ __forceinline__ float group4_max(float v) {
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float group4_sum(float v) {
  v += __shfl_xor(v, 16, 64);
  return v + __shfl_xor(v, 32, 64);
}

template <bool WIDE>
__global__ void __launch_bounds__(512) window_attention_mfma_kernel(MfmaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int H = a.H, G = a.G, dq = a.dq, dv = a.dv, Hp = a.Hp, CG = a.CG;
  const int ldk = dq + 16;                        // padded K row (elements): 8 extra dwords
  const int HpS = Hp + 8;                         // padded row of the mix operand
  constexpr bool wide = WIDE;
  // 16-byte staging loads in flight per thread: what the register budget of the form allows
  constexpr int STG = WIDE ? 5 : 2;
  const int dvw = a.dvw;                          // value slice of a workgroup
  const int dvo = (blockIdx.z % a.ndvs) * dvw;
  const int hbase = ((blockIdx.z / a.ndvs) % a.nhs) * NW;
  const int split = blockIdx.z / (a.ndvs * a.nhs);
  const int dvc = min(dvw, dv - dvo);
  const int dvb = dvc >> 4;
  // the K tiles (score phase) and the transposed V tiles (apply phase) of a key tile are never
  // live together: one region serves both, so every kv head of the tile is staged at once
  u16* Ks = (u16*)smem;                           // [CG][TK][ldk]
  u16* Vt = Ks;                                   // [CG][dvw][40]
  u16* Pm = Ks + CG * max(TK * ldk, dvw * 40) + 512;   // [TQ*TK][Hp] (after 1 KiB of DMA slack)
  // without head mixing neither the mix operand nor the mixing matrix take LDS
  const bool lean = wide || a.talk == nullptr;
  u16* Pp = Pm + (lean ? 0 : TQ * TK * HpS);      // [H][TQ][40] (wide: [NW][TQ][40], by wave)
  u16* Tk = Pp + (wide ? NW : H) * TQ * 40;       // [Hp16][Hp] talk in bf16, zero padded
  int* slot_all = (int*)(Tk + (lean ? 0 : ((H + 15) & ~15) * Hp));   // [TK] or [slot_cap]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int fr = lane & 15, fq = lane >> 4;
  const int s = blockIdx.y;
  const int t0 = a.cu[s] * a.rowmul + blockIdx.x * TQ;
  const int t_end = a.cu[s + 1] * a.rowmul;
  if (t0 >= t_end) return;
  const int nq = min(TQ, t_end - t0);
  const int p0 = a.positions[t0 / a.rowmul];      // positions of a portion are consecutive
  const int p_last = a.rowmul > 1 ? p0 : p0 + nq - 1;
  // the first query's lower bound is the lowest of the tile (window and block alike)
  const int lo = max(max(0, p0 - a.window + 1), a.chunk > 0 ? p0 / a.chunk * a.chunk : 0);
  const int ntiles = (p_last - lo) / TK + 1;
  const int* bt = a.block_tables + (long)s * a.bt_stride;
  const bool rgrp = a.vrows > 0;
  const int hpg = rgrp ? 1 : H / G, Gk = a.Gk, hpk = H / Gk;
  const int row_c = rgrp ? (blockIdx.x * TQ + fr) / a.vrows : 0;   // this lane's row's value group
  const int my_p = a.rowmul > 1 ? p0 : p0 + fr;   // this lane's query position (column fr)
  // key / value heads this workgroup's query heads read: all of them with head mixing, those
  // of its 8 heads in the wide form (the others are not staged)
  const int h_last = min(H, hbase + NW) - 1;
  const int klo = wide ? hbase / hpk : 0, khi = wide ? h_last / hpk + 1 : Gk;
  const int vlo = rgrp ? blockIdx.x * TQ / a.vrows : (wide ? hbase / hpg : 0);
  const int vhi = rgrp ? (blockIdx.x * TQ + nq - 1) / a.vrows + 1 : (wide ? h_last / hpg + 1 : G);
  const int my_clo = a.chunk > 0 ? my_p / a.chunk * a.chunk : 0;      // first key of its block
  const int clo_last = a.chunk > 0 ? p_last / a.chunk * a.chunk : 0;
  const bool my_q = fr < nq;
  const bool has_talk = a.talk != nullptr;
  const int Hp16 = (H + 15) & ~15;

  if (has_talk) {
    for (int i = tid; i < Hp16 * Hp; i += 512) {
      const int h = i / Hp, g = i % Hp;
      Tk[i] = (h < H && g < H) ? f2bf(a.talk[h * H + g]) : (u16)0;
    }
  }
  // zero the mix operand once: head columns [H, Hp) stay zero for the whole kernel
  if (has_talk)
    for (int i = tid; i < TQ * TK * HpS / 2; i += 512) ((uint32_t*)Pm)[i] = 0u;

  float m_run[MAXHW], l_run[MAXHW];
  f32x4 oacc[MAXHW][MAXDVB];
#pragma unroll
  for (int hh = 0; hh < MAXHW; ++hh) {
    m_run[hh] = -INFINITY;
    l_run[hh] = 0.f;
#pragma unroll
    for (int b = 0; b < MAXDVB; ++b) oacc[hh][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  if (a.sink != nullptr && (a.nsplit <= 1 || split == 0)) {
#pragma unroll
    for (int hh = 0; hh < MAXHW; ++hh) {
      const int h = wide ? hbase + wave : wave + hh * NW;
      if (h >= H || (wide && hh)) continue;
      m_run[hh] = a.sink[h] * LOG2E;              // scores live in the log2 domain
      l_run[hh] = 1.f;
    }
  }
  const int nf = dq >> 5;                         // 32-wide K-steps of the score product
  const float scale2 = a.scale * LOG2E;
  int tile_lo = 0, tile_hi = ntiles;
  if (a.nsplit > 1) {
    const int per = (ntiles + a.nsplit - 1) / a.nsplit;
    tile_lo = split * per;
    tile_hi = min(ntiles, tile_lo + per);
  }
  const long stats_base = ((long)s * gridDim.x + blockIdx.x) * a.nsplit;
  if (a.mode == 2) {                              // global max / sum from every split's pair
#pragma unroll
    for (int hh = 0; hh < MAXHW; ++hh) {
      const int h = wide ? hbase + wave : wave + hh * NW;
      if (h >= H || (wide && hh)) continue;
      float M = -INFINITY;
      for (int k2 = 0; k2 < a.nsplit; ++k2)
        M = fmaxf(M, a.stats_ws[(((stats_base + k2) * H + h) * TQ + fr) * 2]);
      float L = 0.f;
      for (int k2 = 0; k2 < a.nsplit; ++k2) {
        const float* pr = a.stats_ws + (((stats_base + k2) * H + h) * TQ + fr) * 2;
        if (pr[0] != -INFINITY) L += pr[1] * __builtin_amdgcn_exp2f(pr[0] - M);
      }
      m_run[hh] = M;
      l_run[hh] = L;
    }
  }
  // without head mixing an unsplit launch needs one pass only (see the score phase)
  // (mode 3: one pass per key split; the split's max / sum go out with its un-normalised
  // partial output and the reduce kernel weighs the splits)
  // (the all-heads form, WIDE = false without mixing, runs it too: 4 heads a wave, each with
  // its own running pair and accumulators, one K staging for every head of the query tile)
  const bool single = (wide && (a.mode == 0 || a.mode == 3)) || (!wide && lean && a.mode == 0);
  const auto si = [&](int hh) { return wide ? 0 : hh; };
  const int pass_lo = (a.mode == 2 || single) ? 1 : 0, pass_hi = a.mode == 1 ? 1 : 2;
  const int rowsT = (int)(a.o_ws_stride / ((long)H * dv));   // rows of a partial-output image
  // staging walks: per-thread start indices and 512-chunk strides, divided once
  const int vcpr = dvc >> 3;
  const int rowB = ldk * 2;                       // bytes of a padded K row in LDS
  const int drow0 = (wave * 1024 + lane * 16) / rowB, drem0 = (wave * 1024 + lane * 16) % rowB;
  const int dq8k = (NW * 1024) / rowB, dr8k = (NW * 1024) % rowB;
  const int vrest0 = tid >> 5, vc0 = vrest0 / vcpr, vch0 = vrest0 % vcpr;
  const int vq16 = 16 / vcpr, vr16 = 16 % vcpr;
  uint4 qcur[4];                                  // prefetched query fragments of head qh
  int qh = -1;
  auto load_q = [&](int h, int f0, uint4* dst) {
    const u16* qrow = a.q + (long)(t0 + fr) * a.ldq + (long)h * dq + fq * 8;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      dst[u] = uint4{0u, 0u, 0u, 0u};
      if (my_q && f0 + u < nf) dst[u] = *reinterpret_cast<const uint4*>(qrow + (f0 + u) * 32);
    }
  };
  const bool slots_once = a.slot_cap >= ntiles * TK;
  if (slots_once) {
    for (int i = tid + tile_lo * TK; i < tile_hi * TK; i += 512) {
      const int j = lo + i;
      slot_all[i] = j <= p_last ? bt[j / a.block_size] * a.block_size + j % a.block_size : -1;
    }
  }

  for (int pass = pass_lo; pass < pass_hi; ++pass) {
    for (int tile = tile_lo; tile < tile_hi; ++tile) {
      const int j0 = lo + tile * TK;
      int* slot = slots_once ? slot_all + tile * TK : slot_all;
      if (!slots_once) {
        __syncthreads();                          // previous tile's readers are done
        if (tid < TK) {
          const int j = j0 + tid;
          slot[tid] = j <= p_last ? bt[j / a.block_size] * a.block_size + j % a.block_size : -1;
        }
      }
      for (int c0 = klo; c0 < khi; c0 += CG) {
        const int cg = min(CG, khi - c0);
        {                                         // this wave's first head of the step: its
          int h0 = -1;                            // query fragments fly with the K tiles
#pragma unroll
          for (int h2 = MAXHW - 1; h2 >= 0; --h2) {
            const int hc = wide ? hbase + wave : wave + h2 * NW;
            if ((!wide || h2 == 0) && hc < H && hc / hpk >= c0 && hc / hpk < c0 + cg) h0 = hc;
          }
          qh = h0;
          if (h0 >= 0) load_q(h0, 0, qcur);
        }
        __syncthreads();                          // slot table ready; Ks free
        {                                         // stage K tiles of kv heads [c0, c0+cg)
          // LDS-DMA (global_load_lds_dwordx4): no staging registers, every piece in flight at
          // once. A wave's instruction fills 1 KiB of the padded row image lane-linearly, so
          // lane L of piece p loads whatever belongs at byte p * 1024 + 16 L: row = that / row
          // bytes, the 16-byte chunk inside the row, or nothing useful in the row's padding
          // and in rows of masked keys (row 0 of the cache: the score is masked anyway).
          const int total_b = cg * TK * rowB;
          int row = drow0, rem = drem0;
          for (int pb = wave * 1024; pb < total_b; pb += NW * 1024) {
            const u16* src = a.k;
            if (row < cg * TK && rem < dq * 2) {
              const int sl = slot[row & (TK - 1)];
              src = a.k + (long)(sl >= 0 ? sl : 0) * a.k_stride + (c0 + (row >> 5)) * dq +
                    (rem >> 1);
            }
            __builtin_amdgcn_global_load_lds((gbl_void*)src, (lds_void*)((char*)Ks + pb), 16, 0, 0);
            row += dq8k;
            rem += dr8k;
            if (rem >= rowB) { rem -= rowB; row += 1; }
          }
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __syncthreads();
#pragma unroll
        for (int hh = 0; hh < MAXHW; ++hh) {
          const int h = wide ? hbase + wave : wave + hh * NW;
          if (h >= H || (wide && hh)) continue;
          const int c = h / hpk;
          if (c < c0 || c >= c0 + cg) continue;
          const u16* kt = Ks + (long)(c - c0) * TK * ldk;
          f32x4 sacc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
          // query fragments, 4 at a time, one group ahead: the next group (of this head, or
          // the first of this wave's next head) is requested before this group's MFMAs
          int hn = -1;                            // this wave's next head of the step
#pragma unroll
          for (int h2 = MAXHW - 1; h2 > hh; --h2) {
            const int hc = wave + h2 * NW;
            if (!wide && hc < H && hc / hpk >= c0 && hc / hpk < c0 + cg) hn = hc;
          }
          if (qh != h) load_q(h, 0, qcur);        // not prefetched (first head of the step)
          for (int f0 = 0; f0 < nf; f0 += 4) {
            uint4 qnxt[4];
            if constexpr (wide) {                 // registers allow the look-ahead only here
              if (f0 + 4 < nf) load_q(h, f0 + 4, qnxt);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              if (f0 + u >= nf) continue;
              const bf16x8 qf = *reinterpret_cast<const bf16x8*>(&qcur[u]);
#pragma unroll
              for (int kb = 0; kb < 2; ++kb) {
                const bf16x8 kf = *reinterpret_cast<const bf16x8*>(
                    kt + (long)(kb * 16 + fr) * ldk + (f0 + u) * 32 + fq * 8);
                sacc[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf, sacc[kb], 0, 0, 0);
              }
            }
            if constexpr (wide) {
#pragma unroll
              for (int u = 0; u < 4; ++u) qcur[u] = qnxt[u];
            } else {
              if (f0 + 4 < nf) load_q(h, f0 + 4, qcur);
              else if (hn >= 0) load_q(hn, 0, qcur);   // next head's first group, under the
            }                                          // softmax arithmetic of this one
          }
          qh = hn;
          // lane: query fr, keys j0 + kb*16 + 4*fq + r. Scores are kept in the log2 domain
          // (scale and slope carry log2 e), so every exponential is one v_exp_f32:
          //   x = s * scale2 - slope2 * (p - j) = fma(s, scale2, slope2 * (j - p))
          const float slope2 = a.slopes ? a.slopes[h] * LOG2E : 0.f;
          const float b0 = slope2 * (float)(j0 + fq * 4 - my_p);
          float sv[8];
          float tmax = -INFINITY;
          // interior tiles (every key visible to every query row): no masking arithmetic
          const bool interior = nq == TQ && j0 + TK - 1 <= p0 && j0 > p_last - a.window &&
                                j0 >= clo_last;
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              float x = fmaf(sacc[kb][r], scale2, b0 + slope2 * (float)(kb * 16 + r));
              if (!interior) {
                const int key = j0 + kb * 16 + fq * 4 + r;
                const int dist = my_p - key;
                if (!my_q || dist < 0 || dist >= a.window || key < my_clo) x = -INFINITY;
              }
              sv[kb * 4 + r] = x;
              tmax = fmaxf(tmax, x);
            }
          if (single) {
            // one pass (no head mixing, so un-normalised weights can be applied at once):
            // running max with the accumulators rescaled when it moves, 1 / l at the end
            tmax = group4_max(tmax);
            const float m_new = fmaxf(m_run[si(hh)], tmax);
            const float mm = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run[si(hh)] - mm);
            float w[8];
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) { w[i] = __builtin_amdgcn_exp2f(sv[i] - mm); sum += w[i]; }
            sum = group4_sum(sum);
            l_run[si(hh)] = l_run[si(hh)] * alpha + sum;
            m_run[si(hh)] = m_new;
            if (alpha != 1.f) {
#pragma unroll
              for (int g2 = 0; g2 < MAXHW; ++g2) {
                if (!wide && g2 != hh) continue;      // this head's accumulators only
#pragma unroll
                for (int b = 0; b < MAXDVB; ++b) oacc[g2][b] *= alpha;
              }
            }
            u16* dst = Pp + ((wide ? wave : h) * TQ + fr) * 40 + fq * 4;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
              uint2 pk;
              pk.x = pack2bf(w[kb * 4], w[kb * 4 + 1]);
              pk.y = pack2bf(w[kb * 4 + 2], w[kb * 4 + 3]);
              *reinterpret_cast<uint2*>(dst + kb * 16) = pk;
            }
          } else if (pass == 0) {
            tmax = group4_max(tmax);
            const float m_new = fmaxf(m_run[hh], tmax);
            // exp2(-inf - m) = 0 for a finite m; a row with no visible key yet keeps m = -inf
            const float mm = m_new == -INFINITY ? 0.f : m_new;
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += __builtin_amdgcn_exp2f(sv[i] - mm);
            sum = group4_sum(sum);
            l_run[hh] = l_run[hh] * __builtin_amdgcn_exp2f(m_run[hh] - mm) + sum;
            m_run[hh] = m_new;
          } else {
            const float inv = l_run[hh] > 0.f ? 1.f / l_run[hh] : 0.f;
            const float mm = m_run[hh] == -INFINITY ? 0.f : m_run[hh];
            float w[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) w[i] = __builtin_amdgcn_exp2f(sv[i] - mm) * inv;
            if (has_talk) {
              // row = key * TQ + query: the 16 queries of a key sit 20 dwords apart
              u16* dst = Pm + (fq * 4 * TQ + fr) * HpS + h;
#pragma unroll
              for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[(kb * 16 + r) * TQ * HpS] = f2bf(w[kb * 4 + r]);
            } else {
              // 4 consecutive keys of one query: one 8-byte store per key block
              u16* dst = Pp + ((wide ? wave : h) * TQ + fr) * 40 + fq * 4;
#pragma unroll
              for (int kb = 0; kb < 2; ++kb) {
                uint2 pk;
                pk.x = pack2bf(w[kb * 4], w[kb * 4 + 1]);
                pk.y = pack2bf(w[kb * 4 + 2], w[kb * 4 + 3]);
                *reinterpret_cast<uint2*>(dst + kb * 16) = pk;
              }
            }
          }
        }
      }
      if (pass == 0) continue;
      if (has_talk) {
        __syncthreads();                          // every head's weights are in Pm
        // W'[h][x] = sum_g talk[h][g] Pm[x][g]: jobs = (h block, x block of 16)
        const int nxb = TQ * TK / 16, jobs = (Hp16 >> 4) * nxb;
        for (int job = wave; job < jobs; job += NW) {
          const int hb = job / nxb, xb = job % nxb;
          f32x4 acc = {0.f, 0.f, 0.f, 0.f};
          for (int kk = 0; kk < Hp; kk += 32) {
            const bf16x8 tf = *reinterpret_cast<const bf16x8*>(
                Tk + (long)(hb * 16 + fr) * Hp + kk + fq * 8);
            const bf16x8 pf = *reinterpret_cast<const bf16x8*>(
                Pm + (long)(xb * 16 + fr) * HpS + kk + fq * 8);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tf, pf, acc, 0, 0, 0);
          }
          // lane: heads hb*16 + 4*fq + r, x = xb*16 + fr  (x = key * TQ + query)
          const int x = xb * 16 + fr, qi = x % TQ, key = x / TQ;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int h = hb * 16 + fq * 4 + r;
            if (h < H) Pp[((long)h * TQ + qi) * 40 + key] = f2bf(acc[r]);
          }
        }
      }
      // O += W' . V per group of kv heads
      for (int c0 = vlo; c0 < vhi; c0 += a.cgv) {
        const int cg = min(a.cgv, vhi - c0);
        __syncthreads();                          // Pp complete (first step) / Vt free
        {
          // chunk i = (c * vcpr + ch) * TK + r: consecutive threads take consecutive keys of one
          // 8-dim chunk, so their transposed 2-byte stores fall into consecutive LDS addresses
          const int total = cg * TK * vcpr;
          const int r = tid & (TK - 1);
          int cc = vc0, ch = vch0;
          for (int base = 0; base < total; base += 512 * STG) {
            uint4 val[STG];
            int lds_off[STG];
#pragma unroll
            for (int u = 0; u < STG; ++u) {
              val[u] = uint4{0u, 0u, 0u, 0u};
              lds_off[u] = -1;
              if (base + u * 512 + tid < total) {
                lds_off[u] = (cc * dvw + ch * 8) * 40 + r;
                const int sl = slot[r];
                if (sl >= 0)
                  val[u] = *reinterpret_cast<const uint4*>(a.v + (long)sl * a.v_stride +
                                                           (c0 + cc) * dv + dvo + ch * 8);
              }
              cc += vq16;
              ch += vr16;
              if (ch >= vcpr) { ch -= vcpr; cc += 1; }
            }
#pragma unroll
            for (int u = 0; u < STG; ++u) {
              if (lds_off[u] >= 0) {
                const u16* e = reinterpret_cast<const u16*>(&val[u]);
                u16* dst = Vt + lds_off[u];
#pragma unroll
                for (int w = 0; w < 8; ++w) dst[w * 40] = e[w];
              }
            }
          }
        }
        __syncthreads();
#pragma unroll
        for (int hh = 0; hh < MAXHW; ++hh) {
          const int h = wide ? hbase + wave : wave + hh * NW;
          if (h >= H) continue;
          const bf16x8 pf = *reinterpret_cast<const bf16x8*>(
              Pp + ((long)(wide ? wave : h) * TQ + fr) * 40 + fq * 8);
          // rows-are-heads with grouped values: every staged group in turn, the weights of
          // the rows of other groups zeroed (operand B's row is this lane's fr)
          const int c_lo = rgrp ? c0 : h / hpg, c_hi = rgrp ? c0 + cg : c_lo + 1;
          if (!rgrp && (c_lo < c0 || c_lo >= c0 + cg)) continue;
          for (int c = c_lo; c < c_hi; ++c) {
            bf16x8 pm = pf;
            if (rgrp && row_c != c) pm = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
            const u16* vt = Vt + (long)(c - c0) * dvw * 40;
#pragma unroll
            for (int b = 0; b < MAXDVB; ++b) {
              const int blk = wide ? hh * MAXDVB + b : b;
              if (blk >= dvb) continue;
              const bf16x8 vf = *reinterpret_cast<const bf16x8*>(vt + (long)(blk * 16 + fr) * 40 + fq * 8);
              // operand A = V^T rows (dim), operand B = W' rows (query): lane holds dims
              // blk*16 + 4*fq + r of query fr
              oacc[hh][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pm, oacc[hh][b], 0, 0, 0);
            }
          }
        }
      }
    }
  }
  if (a.mode == 1) {
    if (fq == 0) {
#pragma unroll
      for (int hh = 0; hh < MAXHW; ++hh) {
        const int h = wide ? hbase + wave : wave + hh * NW;
        if (h >= H || (wide && hh)) continue;
        float* pr = a.stats_ws + (((stats_base + split) * H + h) * TQ + fr) * 2;
        pr[0] = m_run[hh];
        pr[1] = l_run[hh];
      }
    }
    return;
  }
  if (!my_q) return;
  if (a.mode == 3 && fq == 0 && hbase + wave < H) {
    float* pr = a.stats_ws + (((long)split * rowsT + t0 + fr) * H + hbase + wave) * 2;
    pr[0] = m_run[0];
    pr[1] = l_run[0];
  }
  if (a.mode == 2 || a.mode == 3) {
#pragma unroll
    for (int hh = 0; hh < MAXHW; ++hh) {
      const int h = wide ? hbase + wave : wave + hh * NW;
      if (h >= H) continue;
#pragma unroll
      for (int b = 0; b < MAXDVB; ++b) {
        const int blk = wide ? hh * MAXDVB + b : b;
        if (blk >= dvb) continue;
        const int col = h * dv + dvo + blk * 16 + fq * 4;
        *reinterpret_cast<f32x4*>(a.o_ws + (long)split * a.o_ws_stride +
                                  (long)(t0 + fr) * H * dv + col) = oacc[hh][b];
      }
    }
    return;
  }
#pragma unroll
  for (int hh = 0; hh < MAXHW; ++hh) {
    const int h = wide ? hbase + wave : wave + hh * NW;
    if (h >= H) continue;
    const float onorm = single ? (l_run[si(hh)] > 0.f ? 1.f / l_run[si(hh)] : 0.f) : 1.f;
#pragma unroll
    for (int b = 0; b < MAXDVB; ++b) {
      const int blk = wide ? hh * MAXDVB + b : b;
      if (blk >= dvb) continue;
      const int col = h * dv + dvo + blk * 16 + fq * 4;
      float o[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        o[r] = oacc[hh][b][r] * onorm;
        if (a.gate != nullptr)
          o[r] *= 1.f / (1.f + expf(-a.gate[(long)(t0 + fr) * a.ldg + (a.head_gate ? h : col + r)]));
        o[r] *= a.out_scale;
      }
      uint2 pk;
      pk.x = pack2bf(o[0], o[1]);
      pk.y = pack2bf(o[2], o[3]);
      *reinterpret_cast<uint2*>(a.out + (long)(t0 + fr) * a.ldo + col) = pk;
    }
  }
}

// out[t][c] = bf16(gate * sum over splits of the partial outputs), 4 columns a thread
__global__ void __launch_bounds__(256) split_reduce_kernel(
    u16* __restrict__ out, int ldo, const float* __restrict__ o_ws, long stride, int nsplit,
    const float* __restrict__ gate, int ldg, int T, int width, const float* __restrict__ stats,
    int H, int dv, int head_gate, float out_scale) {
  const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int w4 = width >> 2;
  if (gid >= (long)T * w4) return;
  const int t = (int)(gid / w4), c = (int)(gid % w4) * 4;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (stats != nullptr) {
    // un-normalised partials with their own (max, sum) in the log2 domain
    const int h = c / dv;
    float M = -INFINITY, L = 0.f;
    for (int k = 0; k < nsplit; ++k) M = fmaxf(M, stats[(((long)k * T + t) * H + h) * 2]);
    for (int k = 0; k < nsplit; ++k) {
      const float* pr = stats + (((long)k * T + t) * H + h) * 2;
      if (pr[0] == -INFINITY) continue;
      const float wk = __builtin_amdgcn_exp2f(pr[0] - M);
      L += pr[1] * wk;
      acc += wk * *reinterpret_cast<const f32x4*>(o_ws + k * stride + (long)t * width + c);
    }
    acc *= L > 0.f ? 1.f / L : 0.f;
  } else {
    for (int k = 0; k < nsplit; ++k)
      acc += *reinterpret_cast<const f32x4*>(o_ws + k * stride + (long)t * width + c);
  }
  if (gate != nullptr) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      acc[r] *= 1.f / (1.f + expf(-gate[(long)t * ldg + (head_gate ? c / dv : c + r)]));
  }
  acc *= out_scale;
  uint2 pk;
  pk.x = pack2bf(acc[0], acc[1]);
  pk.y = pack2bf(acc[2], acc[3]);
  *reinterpret_cast<uint2*>(out + (long)t * ldo + c) = pk;
}

}  // namespace

// Workspace bytes the key-split form may use for a step of T rows in num_seqs sequences
// (0: the step will not be split).
static int pick_splits(int num_seqs, int max_seqlen, int H, int dv, int window, bool wide) {
  const int qtiles = (max_seqlen + TQ - 1) / TQ;
  const int ndvs = wide ? (dv + 511) / 512 : (dv + 127) / 128, nhs = wide ? (H + NW - 1) / NW : 1;
  const long base = (long)qtiles * num_seqs * ndvs * nhs;
  const int ntiles_max = (window + TQ - 2) / TK + 2;
  if (ntiles_max < 4) return 1;
  // one-pass (wide) launches that just fill the chip with one workgroup per CU still walk
  // their tiles one after the other with nothing to hide the staging behind: split them too
  if (base >= 256 && (!wide || base >= 1024 || ntiles_max < 8)) return 1;
  long n = (base >= 256 ? 1024 : 512) / base;
  if (n > 16) n = 16;
  if (n > ntiles_max / 2) n = ntiles_max / 2;
  return n < 2 ? 1 : (int)n;
}

extern "C" long dli_window_attention_mfma_workspace_bytes(int num_seqs, int max_seqlen, int T,
                                                          int H, int dv, int window,
                                                          int mixing, int rowhead) {
  if (rowhead) {
    max_seqlen = H;
    T *= H;
    H = 1;
  }
  const int nsplit = pick_splits(num_seqs, max_seqlen, H, dv, window, mixing == 0);
  if (nsplit == 1) return 0;
  const long qtiles = (max_seqlen + TQ - 1) / TQ;
  const long st_tiles = (long)num_seqs * qtiles * nsplit * H * TQ * 2;   // two-pass form
  const long st_rows = (long)nsplit * T * H * 2;                          // one-pass form
  return ((st_tiles > st_rows ? st_tiles : st_rows) + (long)nsplit * T * H * dv) * 4;
}

// Returns hipErrorNotSupported (801) when the shapes do not fit this form; the caller then
// runs the scalar kernel.
extern "C" int dli_window_attention_mfma(
    const void* q, int ldq, const void* k, long k_stride, const void* v, long v_stride, void* out,
    int ldo, const float* gate, int ldg, const float* slopes, const float* talk, const int* cu,
    const int* positions, const int* block_tables, int bt_stride, int block_size, int num_seqs,
    int max_seqlen, int H, int G, int dq, int dv, int window, float scale, int T, void* ws,
    int rowhead, int Gk, int chunk, const float* sink, int head_gate, float out_scale,
    hipStream_t st) {
  if (num_seqs <= 0 || max_seqlen <= 0) return 0;
  if (chunk < 0 || Gk < 1) return (int)hipErrorInvalidValue;
  // the sink rides on the one-pass forms' running (max, sum); with head mixing it has no place
  if (sink != nullptr && (talk != nullptr || rowhead)) return (int)hipErrorNotSupported;
  if (head_gate && dv % 4) return (int)hipErrorNotSupported;
  // keys a query tile can see: bounds the slot table and the key splits
  const int weff = chunk > 0 && chunk < window ? chunk : window;
  int rowmul = 1, vrows = 0;
  if (rowhead) {
    if (talk != nullptr || gate != nullptr || slopes != nullptr || Gk != 1 || G < 1 || H % G ||
        max_seqlen != 1 || ldq != H * dq || ldo != H * dv)
      return (int)hipErrorInvalidValue;
    if (G > 1) vrows = H / G;   // grouped values under the shared key row
    rowmul = H;            // token t's heads = rows [t*H, (t+1)*H) of a one-head problem
    max_seqlen = H;
    T *= H;
    ldq = dq;
    ldo = dv;
    H = 1;
  }
  const bool aligned = (uintptr_t)q % 16 == 0 && (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0 &&
                       (uintptr_t)out % 8 == 0 && ldq % 8 == 0 && k_stride % 8 == 0 &&
                       v_stride % 8 == 0 && ldo % 4 == 0;
  bool wide = talk == nullptr;
  // every head scores one shared key row (Gk = 1) and the launch is not split over keys: all
  // heads of a query tile in one workgroup (4 a wave), so the K tile is staged once for them
  // instead of once per 8 heads
  if (wide && !rowhead && Gk == 1 && G > 1 && H > NW && H <= NW * MAXHW &&
      (ws == nullptr || pick_splits(num_seqs, max_seqlen, H, dv, weff, true) == 1))
    wide = false;
  const bool lean = talk == nullptr;
  if (H < 1 || (!wide && H > NW * MAXHW) || G < 1 || (vrows == 0 && H % G) || H % Gk || dq % 32 || dv % 16 ||
      !aligned || window < 1 || block_size < 1 || (talk != nullptr && Gk != G))
    return (int)hipErrorNotSupported;
  const int dvw = wide ? (dv >= 512 ? 512 : ((dv + 15) & ~15)) : 128;
  const int Hp = (H + 31) & ~31, Hp16 = (H + 15) & ~15;
  const int ldk = dq + 16;
  // the whole window's cache rows in LDS when they take at most 16 KB
  int slot_cap = ((weff + TQ - 2) / TK + 2) * TK;
  if ((size_t)slot_cap * 4 > 16 * 1024) slot_cap = 0;
  const size_t fixed = (wide ? (size_t)NW * TQ * 40
                        : lean ? (size_t)H * TQ * 40
                               : (size_t)TQ * TK * (Hp + 8) + (size_t)H * TQ * 40 + (size_t)Hp16 * Hp) * 2 +
                       (size_t)(slot_cap > TK ? slot_cap : TK) * 4 + 64 + 1024;
  const size_t per_cg = (size_t)((TK * ldk > dvw * 40) ? TK * ldk : dvw * 40) * 2;
  const size_t budget = 158 * 1024;
  if (fixed + per_cg > budget) return (int)hipErrorNotSupported;
  int CG = (int)((budget - fixed) / per_cg);
  CG = CG > (G > Gk ? G : Gk) ? (G > Gk ? G : Gk) : CG;
  CG = CG > NW ? NW : CG;
  // a wide workgroup's 8 heads read at most this many key / value heads
  if (wide && !rowhead) {
    const int hk = H / Gk, hv = H / G;
    const int need = (NW - 1) / (hk < hv ? hk : hv) + 2;
    CG = CG > need ? need : CG;
  }
  int cgv = (int)(CG * (per_cg / 2) / ((size_t)dvw * 40));   // value groups that fit the regions
  cgv = cgv > G ? G : cgv;
  const size_t sh = fixed + CG * per_cg;
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void*)window_attention_mfma_kernel<false>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)window_attention_mfma_kernel<true>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return (int)e;
    raised = true;
  }
#define WA_LAUNCH(GRID)                                                           \
  do {                                                                            \
    if (wide) window_attention_mfma_kernel<true><<<GRID, 512, sh, st>>>(a);       \
    else window_attention_mfma_kernel<false><<<GRID, 512, sh, st>>>(a);           \
  } while (0)
  const int ndvs = (dv + dvw - 1) / dvw, qtiles = (max_seqlen + TQ - 1) / TQ;
  const int nhs = wide ? (H + NW - 1) / NW : 1;
  // (the all-heads form was chosen because the launch needs no key split)
  const int nsplit = ws != nullptr && !(lean && !wide)
                         ? pick_splits(num_seqs, max_seqlen, H, dv, weff, wide) : 1;
  MfmaArgs a{(const u16*)q, ldq, (const u16*)k, k_stride, (const u16*)v, v_stride, (u16*)out,
             ldo, gate, ldg, slopes, talk, cu, positions, block_tables, bt_stride, block_size,
             H, G, dq, dv, window, scale, Gk, chunk, Hp, CG, 0, 1, ndvs, wide ? 1 : 0, nhs, rowmul,
             vrows, cgv, slot_cap, sink, head_gate, out_scale, dvw, nullptr, nullptr, 0};
  if (nsplit == 1) {
    dim3 grid(qtiles, num_seqs, ndvs * nhs);
    WA_LAUNCH(grid);
    DLI_RETURN_LAUNCH();
  }
  if (T <= 0 || (H * dv) % 4 || ldo % 4) return (int)hipErrorInvalidValue;
  a.nsplit = nsplit;
  a.stats_ws = (float*)ws;
  {
    const long st_tiles = (long)num_seqs * qtiles * nsplit * H * TQ * 2;
    const long st_rows = (long)nsplit * T * H * 2;
    a.o_ws = a.stats_ws + (st_tiles > st_rows ? st_tiles : st_rows);
  }
  a.o_ws_stride = (long)T * H * dv;
  const long quads = (long)T * (H * dv / 4);
  if (wide) {            // no mixing: one pass per split, the reduce weighs the splits
    a.mode = 3;
    WA_LAUNCH(dim3(qtiles, num_seqs, ndvs * nhs * nsplit));
    split_reduce_kernel<<<(int)((quads + 255) / 256), 256, 0, st>>>(
        (u16*)out, ldo, a.o_ws, a.o_ws_stride, nsplit, gate, ldg, T, H * dv, a.stats_ws, H, dv,
        head_gate, out_scale);
    DLI_RETURN_LAUNCH();
  }
  a.mode = 1;
  a.ndvs = 1;                                     // the statistics do not depend on the slice
  WA_LAUNCH(dim3(qtiles, num_seqs, nhs * nsplit));
  a.mode = 2;
  a.ndvs = ndvs;
  WA_LAUNCH(dim3(qtiles, num_seqs, ndvs * nhs * nsplit));
  split_reduce_kernel<<<(int)((quads + 255) / 256), 256, 0, st>>>(
      (u16*)out, ldo, a.o_ws, a.o_ws_stride, nsplit, gate, ldg, T, H * dv, nullptr, H, dv,
      head_gate, out_scale);
  DLI_RETURN_LAUNCH();
}
