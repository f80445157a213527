// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Softmax attention with grouped keys / values over a paged cache, with a sliding window that also keeps the
// sequence's first tokens (models/suvapel.py):
//
//   visible(p, j) = j <= p and (p - j < window or j < keep_first)      (window 0: every j <= p)
//   a kept key is rotated and masked by the position it was written at, like any other key;
//   head h's result is multiplied by sigmoid(gate[t, h]), one number per token and head (gate null: none).
//   With `dist` (three numbers r1, r2, pb per head) there is no softmax: the weight of a visible key is
//   sigmoid(score - r1 log(1 + r2 (p - j)) + pb), a logarithmic distance bias taken off the score, and the
//   weights are summed against the values as they are.
//
// `rope_append`: rows [q (H x D) | k (G x D) | v (G x Dv)] -> q [T, H, D]; with q_norm / k_norm [D] every q / k
// head is first divided by its root mean square (eps inside the root) and multiplied by that weight (one workgroup
// per token, a wave per head); rotary positions on the first `rot`
// entries of every q and k head (pairs (i, i + rot/2), angle = position * inv_freq[i] in fp32, cos and sin times
// `mag`: a frequency table and a magnitude are what YaRN-style scalings come down to); the rotated keys and the
// values go to the paged cache.  Cache layout: k_cache [NB, G, BS, D] (token-major), v_cache [NB, G, Dv, BS] (a page's
// values of one entry contiguous); slot = page * BS + offset (-1: a padding row, nothing is written or attended).
//
// `sliding_attention`, vector kernel: one workgroup per (token, key/value head) with the H / G query heads that
// share it (or as many of them as its accumulators hold; the rest go to further workgroups).  The visible keys (the kept first ones, then the window) are walked in page-aligned tiles of 64
// positions with an online softmax: scores by one thread per (query head, key), the tile's maximum / sum per head by
// one wave, weights x values by one thread per output entry, a page's values in 16-byte pieces.  Scores, weights and all sums are fp32; AT (bf16_t or float) is the type
// of q, the cache, the gate and the output.  A decode step is the same launch with one token per sequence, so a
// position's result does not depend on whether it was a prompt row or a decoded one.
#include "attention_window.h"

namespace {
using namespace rows;

constexpr int KT = 64;        // keys per tile
constexpr int MAX_REP = 16;   // query heads per key/value head
constexpr int MAX_ACC = 8;    // output entries per thread: (H / G) * Dv <= NT * MAX_ACC
constexpr int TILE_MIN_ROWS = 8;   // steps whose longest run of rows is shorter stay on the vector kernel

template <typename AT>
__global__ __launch_bounds__(NT) void rope_append_kernel(AT* __restrict__ q_out, const AT* __restrict__ qkv,
                                                         const float* __restrict__ inv_freq, float mag,
                                                         const int* __restrict__ positions, const int* __restrict__ slots,
                                                         AT* __restrict__ k_cache, AT* __restrict__ v_cache, int H, int G,
                                                         int D, int Dv, int rot, int BS, const float* __restrict__ q_norm,
                                                         const float* __restrict__ k_norm, float eps) {
  extern __shared__ float hinv[];   // [H + G] 1 / rms of each q and k head (only with a norm)
  const int t = blockIdx.x;
  const int half = rot >> 1;
  const float pos = (float)positions[t];
  const int slot = slots[t];
  const AT* row = qkv + (size_t)t * ((H + G) * D + G * Dv);
  const size_t page = slot >= 0 ? (size_t)(slot / BS) : 0, offs = slot >= 0 ? (size_t)(slot % BS) : 0;
  const bool normed = q_norm != nullptr || k_norm != nullptr;
  if (normed) {
    const int lane = threadIdx.x & 63;
    for (int hh = threadIdx.x >> 6; hh < H + G; hh += NW) {
      float s = 0.f;
      for (int i = lane; i < D; i += 64) {
        const float v = ldf(row + hh * D + i);
        s += v * v;
      }
      s = wave_sum(s);
      if (lane == 0) hinv[hh] = (hh < H ? q_norm : k_norm) != nullptr ? 1.0f / sqrtf(s / (float)D + eps) : 1.0f;
    }
    __syncthreads();
  }
  for (int idx = threadIdx.x; idx < (H + G) * D; idx += NT) {
    const int hh = idx / D, i = idx % D;
    if (hh >= H && slot < 0) break;
    float o = ldf(row + idx);
    const float* nw = hh < H ? q_norm : k_norm;
    if (nw != nullptr) o *= hinv[hh] * nw[i];
    if (i < rot) {
      const int j = i < half ? i : i - half;
      const int pi = i < half ? i + half : i - half;
      float partner = ldf(row + hh * D + pi);
      if (nw != nullptr) partner *= hinv[hh] * nw[pi];
      float sn, cs;
      sincosf(pos * inv_freq[j], &sn, &cs);
      sn *= mag;
      cs *= mag;
      o = i < half ? o * cs - partner * sn : o * cs + partner * sn;
    }
    if (hh < H) stf(q_out + (size_t)t * H * D + idx, o);
    else stf(k_cache + ((page * G + (hh - H)) * BS + offs) * D + i, o);
  }
  if (slot < 0) return;
  const AT* vrow = row + (H + G) * D;
  for (int idx = threadIdx.x; idx < G * Dv; idx += NT)
    v_cache[((page * G + idx / Dv) * Dv + idx % Dv) * BS + offs] = vrow[idx];
}


template <typename AT>
__global__ __launch_bounds__(NT) void sliding_attention_kernel(AT* __restrict__ out, const AT* __restrict__ q,
                                                               const AT* __restrict__ k_cache,
                                                               const AT* __restrict__ v_cache, const AT* __restrict__ gate,
                                                               SlideArgs a, int hpw) {
  extern __shared__ float lds[];
  const int H = a.H, G = a.G, D = a.D, Dv = a.Dv, BS = a.BS;
  // the workgroup's query heads: `hpw` of the H / G heads of key/value head g, from head g * (H / G) + hb on
  const int hb = blockIdx.z * hpw, rep = min(hpw, H / G - hb), h0 = blockIdx.y * (H / G) + hb;
  float* qs = lds;                  // [rep * D]
  float* sc = qs + rep * D;         // [rep * KT] scores, then weights of the tile
  __shared__ float s_m[MAX_REP], s_l[MAX_REP], s_c[MAX_REP];   // running maximum, running sum, the tile's rescale
  __shared__ int s_page[KT];        // (page * G + g) of each page of the tile (KT / BS of them)
  const int t = blockIdx.x, g = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int RV = rep * Dv;
  AT* orow = out + ((size_t)t * H + h0) * Dv;
  if (a.slots[t] < 0 || (a.q_starts != nullptr && t >= a.q_starts[a.num_seqs])) {
    for (int i = threadIdx.x; i < RV; i += NT) stf(orow + i, 0.f);
    return;
  }
  const int p = a.positions[t];
  const int seq = seq_of(a.q_starts, a.num_seqs, t);
  const int* bt = a.block_tables + (size_t)seq * a.max_blocks;
  const int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;   // first position of the window
  const int nk0 = min(a.keep_first, lo);                        // kept first positions that lie before the window
  for (int i = threadIdx.x; i < rep * D; i += NT) qs[i] = ldf(q + ((size_t)t * H + h0) * D + i);
  const bool sig = a.dist != nullptr;
  if (threadIdx.x < rep) {   // sigmoid weights are final as they are: no maximum, no rescale, no denominator
    s_m[threadIdx.x] = -INFINITY;
    s_l[threadIdx.x] = sig ? 1.f : 0.f;
    s_c[threadIdx.x] = 1.f;
  }
  float acc[MAX_ACC];
#pragma unroll
  for (int u = 0; u < MAX_ACC; ++u) acc[u] = 0.f;
  // two spans of positions: the kept first ones [0, nk0), then the window [lo, p]; each is walked in tiles of KT
  // positions that start on a page border, the positions of a tile outside its span are masked
  for (int span = 0; span < 2; ++span) {
    const int sa = span == 0 ? 0 : lo, sb = span == 0 ? nk0 : p + 1;
    for (int pos0 = (sa / BS) * BS; pos0 < sb; pos0 += KT) {
      __syncthreads();
      if (threadIdx.x < KT / BS && pos0 + threadIdx.x * BS < sb) s_page[threadIdx.x] = bt[pos0 / BS + threadIdx.x] * G + g;
      __syncthreads();
      for (int it = threadIdx.x; it < rep * KT; it += NT) {
        const int r = it / KT, j = it % KT;
        const int pos = pos0 + j;
        float s = -INFINITY;
        if (pos >= sa && pos < sb) {
          const AT* kr = k_cache + ((size_t)s_page[j / BS] * BS + j % BS) * D;
          const float* qg = qs + r * D;
          s = 0.f;
          if constexpr (sizeof(AT) == 2) {
            if ((D & 7) == 0) {   // 16-byte loads: 8 bf16 key entries against 8 fp32 query entries from LDS
              for (int i = 0; i < D; i += 8) {
                const uint4 kv = *reinterpret_cast<const uint4*>(kr + i);
                const f32x4 qa = *reinterpret_cast<const f32x4*>(qg + i), qb = *reinterpret_cast<const f32x4*>(qg + i + 4);
                s += qa[0] * lo_f(kv.x) + qa[1] * hi_f(kv.x) + qa[2] * lo_f(kv.y) + qa[3] * hi_f(kv.y) +
                     qb[0] * lo_f(kv.z) + qb[1] * hi_f(kv.z) + qb[2] * lo_f(kv.w) + qb[3] * hi_f(kv.w);
              }
            } else {
              for (int i = 0; i < D; ++i) s += qg[i] * ldf(kr + i);
            }
          } else {
            if ((D & 3) == 0) {
              for (int i = 0; i < D; i += 4) {
                const f32x4 kv = *reinterpret_cast<const f32x4*>(kr + i);
                const f32x4 qa = *reinterpret_cast<const f32x4*>(qg + i);
                s += qa[0] * kv[0] + qa[1] * kv[1] + qa[2] * kv[2] + qa[3] * kv[3];
              }
            } else {
              for (int i = 0; i < D; ++i) s += qg[i] * ldf(kr + i);
            }
          }
          s *= a.scale;
          if (sig) s = dist_sigmoid(s, a.dist[h0 + r], a.dist[H + h0 + r], a.dist[2 * H + h0 + r], p - pos);
        } else if (sig) {
          s = 0.f;
        }
        sc[it] = s;
      }
      __syncthreads();
      for (int r = wave; r < rep && !sig; r += NW) {      // the tile's place in head r's running softmax
        const float s = sc[r * KT + lane];
        const float mo = s_m[r];
        const float m = fmaxf(mo, wave_max(s));   // finite: a tile holds at least one position of its span
        const float e = s == -INFINITY ? 0.f : expf(s - m);
        const float sum = wave_sum(e);
        sc[r * KT + lane] = e;
        if (lane == 0) {
          const float corr = mo == -INFINITY ? 0.f : expf(mo - m);
          s_c[r] = corr;
          s_l[r] = s_l[r] * corr + sum;
          s_m[r] = m;
        }
      }
      __syncthreads();
      const int j0 = max(sa - pos0, 0), j1 = min(sb - pos0, KT);   // the tile's positions inside the span
#pragma unroll
      for (int u = 0; u < MAX_ACC; ++u) {
        const int i = threadIdx.x + u * NT;
        if (i < RV) {
          const int r = i / Dv, d = i % Dv;
          const float* wr = sc + r * KT;
          float s = acc[u] * s_c[r];
          if (sizeof(AT) == 2 && BS == 16) {     // a page's 16 values of entry d: two 16-byte loads
            for (int pg = j0 / 16; pg * 16 < j1; ++pg) {
              const uint4* vp = reinterpret_cast<const uint4*>(v_cache + ((size_t)s_page[pg] * Dv + d) * 16);
              const uint4 va = vp[0], vb = vp[1];
              const uint32_t w8[8] = {va.x, va.y, va.z, va.w, vb.x, vb.y, vb.z, vb.w};
              const float* wp = wr + pg * 16;
#pragma unroll
              for (int k = 0; k < 8; ++k) {      // a weight of 0 (outside the span) takes nothing from its slot
                const float w0 = wp[2 * k], w1 = wp[2 * k + 1];
                s += w0 != 0.f ? w0 * lo_f(w8[k]) : 0.f;
                s += w1 != 0.f ? w1 * hi_f(w8[k]) : 0.f;
              }
            }
          } else {
            for (int j = j0; j < j1; ++j) s += wr[j] * ldf(v_cache + ((size_t)s_page[j / BS] * Dv + d) * BS + j % BS);
          }
          acc[u] = s;
        }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < MAX_ACC; ++u) {
    const int i = threadIdx.x + u * NT;
    if (i < RV) {
      const int r = i / Dv;
      float o = acc[u] / s_l[r];
      if (gate != nullptr) o *= 1.0f / (1.0f + expf(-ldf(gate + (size_t)t * a.gs + a.g_off + h0 + r)));
      stf(orow + i, o);
    }
  }
}

}  // namespace

extern "C" int ka_rope_append(void* q_out, const void* qkv, const float* inv_freq, float mag, const int* positions,
                              const int* slots, void* k_cache, void* v_cache, int T, int H, int G, int D, int Dv, int rot,
                              int BS, const float* q_norm, const float* k_norm, float eps, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (D <= 0 || Dv <= 0 || rot < 0 || rot > D || (rot & 1) || BS <= 0 || H <= 0 || G <= 0 || (rot > 0 && inv_freq == nullptr))
    return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(H + G) * sizeof(float);
  if (lds > 32 * 1024) return (int)hipErrorInvalidValue;
  if (f32)
    rope_append_kernel<float><<<T, NT, lds, st>>>((float*)q_out, (const float*)qkv, inv_freq, mag, positions, slots,
                                                  (float*)k_cache, (float*)v_cache, H, G, D, Dv, rot, BS, q_norm, k_norm, eps);
  else
    rope_append_kernel<bf16_t><<<T, NT, lds, st>>>((bf16_t*)q_out, (const bf16_t*)qkv, inv_freq, mag, positions, slots,
                                                   (bf16_t*)k_cache, (bf16_t*)v_cache, H, G, D, Dv, rot, BS, q_norm, k_norm,
                                                   eps);
  KA_CHECK_LAUNCH();
}

// mode: the longest run of rows that one sequence brings to the step (1 for single rows), or 0 to ask for the vector kernel
extern "C" int ka_sliding_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                    const int* block_tables, const int* q_starts, int num_seqs, const int* positions,
                                    const int* slots, const void* gate, int gs, int g_off, int T, int H, int G, int D,
                                    int Dv, int window, int keep_first, int BS, int max_blocks, float scale,
                                    const float* dist, int f32, int mode, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || Dv > NT * MAX_ACC || D <= 0 || Dv <= 0 || BS <= 0 || window < 0 || keep_first < 0 ||
      num_seqs <= 0)
    return (int)hipErrorInvalidValue;
  if (KT % BS) return (int)hipErrorInvalidValue;   // tiles are whole pages
  if (q_starts == nullptr && T > num_seqs) return (int)hipErrorInvalidValue;   // row t reads block-table row t
  SlideArgs a{block_tables, q_starts, positions, slots, num_seqs, H, G, D, Dv, window, keep_first, BS, max_blocks, gs, g_off, scale, dist};
  // bf16 on the matrix cores where the shape allows: prompt portions (mode = the longest run of rows of one
  // sequence in the step) and single rows (q_starts null); mode 0 asks for the vector kernel
  if (!f32 && mode > 0 && (q_starts == nullptr || mode >= TILE_MIN_ROWS) && ka_sliding_attention_tile_ok(H, G, D, Dv, BS))
    return sliding_attention_tile((bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                                  (const bf16_t*)gate, a, mode, T, st);
  // query heads per workgroup: as many of a group's heads as the per-thread accumulators and the LDS hold
  int rep = H / G;
  rep = rep > MAX_REP ? MAX_REP : rep;
  rep = rep * Dv > NT * MAX_ACC ? NT * MAX_ACC / Dv : rep;
  while (rep > 1 && (size_t)(rep * D + rep * KT) * sizeof(float) > 60 * 1024) --rep;
  const size_t lds = (size_t)(rep * D + rep * KT) * sizeof(float);
  if (lds > 60 * 1024) return (int)hipErrorInvalidValue;
  if (lds > 48 * 1024) {
    const void* fn = f32 ? reinterpret_cast<const void*>(sliding_attention_kernel<float>)
                         : reinterpret_cast<const void*>(sliding_attention_kernel<bf16_t>);
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  const dim3 grid(T, G, (H / G + rep - 1) / rep);
  if (f32)
    sliding_attention_kernel<float><<<grid, NT, lds, st>>>((float*)out, (const float*)q, (const float*)k_cache,
                                                           (const float*)v_cache, (const float*)gate, a, rep);
  else
    sliding_attention_kernel<bf16_t><<<grid, NT, lds, st>>>((bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache,
                                                            (const bf16_t*)v_cache, (const bf16_t*)gate, a, rep);
  KA_CHECK_LAUNCH();
}
