// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Latent attention over a paged cache (models/kafilorn.py).  A token's cache entry is one row
// [R + Dr]: the RMS-normed key/value latent c [R] and one rotated key part k_r [Dr] shared by all heads;
// the per-head keys W_uk c and values W_uv c are never materialised: the query is carried into the latent
// space (q_lat = W_uk^T q, a batched GEMM outside), the attention runs multi-query over the rows with the
// latent itself as the value, and W_uv is applied to the result (another batched GEMM outside).
//
//   latent_prep:   from the fused down-projection row [Q | R | Dr]: the RMS-normed query latent [Q] (Q = 0: a
//                  model that projects its queries directly has none); the RMS-normed c and the rotated k_r
//                  appended to the cache at the token's slot.
//   rope_split_q:  q [T, H, D + Dr] (columns `off` .. of rows of P entries, so it may be a part of a fused
//                  projection) -> the unrotated parts [H, T, D] (the batched GEMM's operand layout) and
//                  the rotated parts [T, H, Dr] in fp32.  Rotary: among the first `dims` entries, entry i pairs
//                  with i + dims/2, or (interleaved) entry 2i with 2i + 1; angle = position * inv_freq[i], cos and
//                  sin times `mag` (a frequency table and a magnitude are what YaRN-style scalings come down to).
//   head_gate:     o [H, T, Dv] (the batched value up-projection's result) -> [T, H * Dv], head h times
//                  sigmoid(gate[t, h]) (gate null: the layout change only).
//   window_attention:  s_h(j) = (q_lat_h . c_j + q_rot_h . k_r,j) * scale for the keys j with
//                  0 <= p - j < window (window 0: all j <= p); weights exp(s) / (sum exp(s) + exp(sink_h)),
//                  the sink optional; out_h = sum_j w_h(j) c_j, written [H, T, R].
//                  Any dtype and shape: one workgroup per (token, group of heads), keys in tiles of 64 with an
//                  online softmax in fp32 (mode 1, and what the matrix-core kernel below does not take).  A
//                  decode step is the same launch with one token per sequence.
#include "rows_f32.h"

namespace {
using namespace rows;

constexpr int KT = 64;
constexpr int MAX_ACC = 32;   // outputs per thread: heads per workgroup * R <= NT * MAX_ACC

KA_DEV float rot_entry(float self, float partner, bool first_half, float ang, float mag) {
  float sn, cs;
  sincosf(ang, &sn, &cs);
  sn *= mag;
  cs *= mag;
  return first_half ? self * cs - partner * sn : self * cs + partner * sn;
}

// entry e (< dims) of a rotated vector, given the entry it is paired with (rot_partner)
KA_DEV float rot_at(float self, float partner, int e, int dims, bool interleaved, float pos, const float* inv_freq,
                    float mag) {
  const int half = dims >> 1;
  const bool first = interleaved ? (e & 1) == 0 : e < half;
  const int j = interleaved ? e >> 1 : (e < half ? e : e - half);
  return rot_entry(self, partner, first, pos * inv_freq[j], mag);
}
KA_DEV int rot_partner(int e, int dims, bool interleaved) {
  const int half = dims >> 1;
  return interleaved ? e ^ 1 : (e < half ? e + half : e - half);
}

template <typename AT>
__global__ __launch_bounds__(NT) void latent_prep_kernel(AT* __restrict__ cq, const AT* __restrict__ proj, int P, int Q,
                                                         int R, int Dr, const float* __restrict__ w_q,
                                                         const float* __restrict__ w_kv, const float* __restrict__ inv_freq,
                                                         const int* __restrict__ positions, const int* __restrict__ slots,
                                                         AT* __restrict__ cache, int rot_dims, float eps,
                                                         int interleaved, float mag) {
  __shared__ float red[NW];
  const int t = blockIdx.x;
  const AT* row = proj + (size_t)t * P;
  float s = 0.f, inv;
  if (Q > 0) {
    for (int i = threadIdx.x; i < Q; i += NT) {
      const float v = ldf(row + i);
      s += v * v;
    }
    inv = 1.0f / sqrtf(block_sum(s, red) / (float)Q + eps);
    for (int i = threadIdx.x; i < Q; i += NT) stf(cq + (size_t)t * Q + i, ldf(row + i) * inv * w_q[i]);
  }
  if (cache == nullptr) return;
  const int slot = slots[t];
  if (slot < 0) return;
  s = 0.f;
  for (int i = threadIdx.x; i < R; i += NT) {
    const float v = ldf(row + Q + i);
    s += v * v;
  }
  inv = 1.0f / sqrtf(block_sum(s, red) / (float)R + eps);
  AT* dst = cache + (size_t)slot * (R + Dr);
  for (int i = threadIdx.x; i < R; i += NT) stf(dst + i, ldf(row + Q + i) * inv * w_kv[i]);
  const float pos = (float)positions[t];
  const AT* kr = row + Q + R;
  for (int i = threadIdx.x; i < Dr; i += NT) {
    float o = ldf(kr + i);
    if (i < rot_dims) {
      const float pr = ldf(kr + rot_partner(i, rot_dims, interleaved));
      o = rot_at(o, pr, i, rot_dims, interleaved, pos, inv_freq, mag);
    }
    stf(dst + R + i, o);
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void rope_split_q_kernel(AT* __restrict__ qn, float* __restrict__ qr,
                                                          const AT* __restrict__ q, int P, int off,
                                                          const float* __restrict__ inv_freq,
                                                          const int* __restrict__ positions, int T, int H, int D, int Dr,
                                                          int rot_dims, int interleaved, float mag) {
  const int t = blockIdx.x;
  const int DD = D + Dr;
  const float pos = (float)positions[t];
  const AT* row = q + (size_t)t * P + off;
  for (int idx = threadIdx.x; idx < H * DD; idx += NT) {
    const int h = idx / DD, i = idx % DD;
    if (i < D) {
      qn[((size_t)h * T + t) * D + i] = row[idx];
    } else {
      const int e = i - D;
      float o = ldf(row + idx);
      if (e < rot_dims) {
        const float pr = ldf(row + h * DD + D + rot_partner(e, rot_dims, interleaved));
        o = rot_at(o, pr, e, rot_dims, interleaved, pos, inv_freq, mag);
      }
      qr[((size_t)t * H + h) * Dr + e] = o;
    }
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void head_gate_kernel(AT* __restrict__ out, const AT* __restrict__ o,
                                                       const AT* __restrict__ gate, int gs, int g_off, int T, int H,
                                                       int Dv) {
  const int t = blockIdx.x;
  for (int idx = threadIdx.x; idx < H * Dv; idx += NT) {
    const int h = idx / Dv, d = idx - h * Dv;
    float v = ldf(o + ((size_t)h * T + t) * Dv + d);
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-ldf(gate + (size_t)t * gs + g_off + h)));
    stf(out + (size_t)t * H * Dv + idx, v);
  }
}

struct WinArgs {
  const int* block_tables;   // [S, max_blocks]
  const int* q_starts;       // [S + 1] or null
  int num_seqs;
  const int* positions;      // [T]
  const int* slots;          // [T] < 0: padding row
  const float* sink;         // [H] or null
  int T, H, HG, R, Dr, BS, max_blocks, window;
  float scale;
};

template <typename AT>
__global__ __launch_bounds__(NT) void window_attention_kernel(AT* __restrict__ out, const AT* __restrict__ q_lat,
                                                              const float* __restrict__ q_rot,
                                                              const AT* __restrict__ cache, WinArgs a) {
  extern __shared__ float lds[];
  const int R = a.R, Dr = a.Dr, E = R + Dr, HG = a.HG, H = a.H, T = a.T;
  float* ql = lds;                 // [HG][E]  query in the latent space, then its rotated part
  float* sc = ql + HG * E;         // [HG][KT] scores, then unnormalised weights of the tile
  float* corr = sc + HG * KT;      // [HG] rescale of the accumulators for the tile
  float* linv = corr + HG;         // [HG] 1 / denominator at the end
  __shared__ int page[KT];
  const int t = blockIdx.x, h0 = blockIdx.y * HG;
  const int hg = min(HG, H - h0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (a.slots[t] < 0) {
    for (int i = threadIdx.x; i < hg * R; i += NT) stf(out + ((size_t)(h0 + i / R) * T + t) * R + i % R, 0.f);
    return;
  }
  const int p = a.positions[t];
  const int seq = seq_of(a.q_starts, a.num_seqs, t);
  const int* bt = a.block_tables + (size_t)seq * a.max_blocks;
  const int start = a.window > 0 ? max(0, p - a.window + 1) : 0;
  const int n = p - start + 1;
  for (int i = threadIdx.x; i < hg * E; i += NT) {
    const int g = i / E, e = i % E;
    ql[i] = e < R ? ldf(q_lat + ((size_t)(h0 + g) * T + t) * R + e) : q_rot[((size_t)t * H + h0 + g) * Dr + e - R];
  }
  // running maximum and denominator per head live in the registers of the head's wave (head g: wave g % NW)
  float run_m[16], run_l[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int g = wave + u * NW;
    const bool sk = a.sink != nullptr && g < hg;
    run_m[u] = sk ? a.sink[h0 + g] : -INFINITY;
    run_l[u] = sk ? 1.f : 0.f;
  }
  float acc[MAX_ACC];
#pragma unroll
  for (int u = 0; u < MAX_ACC; ++u) acc[u] = 0.f;
  const int BS = a.BS;
  for (int k0 = 0; k0 < n; k0 += KT) {
    const int nk = min(KT, n - k0);
    __syncthreads();
    if (threadIdx.x < nk) page[threadIdx.x] = bt[(start + k0 + threadIdx.x) / BS];
    __syncthreads();
    for (int it = threadIdx.x; it < hg * KT; it += NT) {
      const int g = it / KT, j = it % KT;
      float s = -INFINITY;
      if (j < nk) {
        const int pos = start + k0 + j;
        const AT* kr = cache + ((size_t)page[j] * BS + pos % BS) * E;
        const float* qg = ql + g * E;
        s = 0.f;
        if constexpr (sizeof(AT) == 2) {
          if ((E & 7) == 0) {
            for (int i = 0; i < E; i += 8) {
              const uint4 kv = *reinterpret_cast<const uint4*>(kr + i);
              const f32x4 qa = *reinterpret_cast<const f32x4*>(qg + i), qb = *reinterpret_cast<const f32x4*>(qg + i + 4);
              s += qa[0] * lo_f(kv.x) + qa[1] * hi_f(kv.x) + qa[2] * lo_f(kv.y) + qa[3] * hi_f(kv.y) +
                   qb[0] * lo_f(kv.z) + qb[1] * hi_f(kv.z) + qb[2] * lo_f(kv.w) + qb[3] * hi_f(kv.w);
            }
          } else {
            for (int i = 0; i < E; ++i) s += qg[i] * ldf(kr + i);
          }
        } else {
          if ((E & 3) == 0) {
            for (int i = 0; i < E; i += 4) {
              const f32x4 kv = *reinterpret_cast<const f32x4*>(kr + i);
              const f32x4 qa = *reinterpret_cast<const f32x4*>(qg + i);
              s += qa[0] * kv[0] + qa[1] * kv[1] + qa[2] * kv[2] + qa[3] * kv[3];
            }
          } else {
            for (int i = 0; i < E; ++i) s += qg[i] * ldf(kr + i);
          }
        }
        s *= a.scale;
      }
      sc[it] = s;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int g = wave + u * NW;
      if (g < hg) {
        const float s = sc[g * KT + lane];
        const float m = fmaxf(run_m[u], wave_max(s));
        const float e = s == -INFINITY ? 0.f : expf(s - m);
        const float c = run_m[u] == -INFINITY ? 0.f : expf(run_m[u] - m);
        run_l[u] = run_l[u] * c + wave_sum(e);
        run_m[u] = m;
        sc[g * KT + lane] = e;
        if (lane == 0) corr[g] = c;
      }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < MAX_ACC; ++u) {
      const int i = threadIdx.x + u * NT;
      if (i < hg * R) {
        const int g = i / R, r = i % R;
        const float* wg = sc + g * KT;
        float s = acc[u] * corr[g];
        for (int j = 0; j < nk; ++j) {
          const int pos = start + k0 + j;
          s += wg[j] * ldf(cache + ((size_t)page[j] * BS + pos % BS) * E + r);
        }
        acc[u] = s;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int g = wave + u * NW;
    if (g < hg && lane == 0) linv[g] = 1.0f / run_l[u];
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < MAX_ACC; ++u) {
    const int i = threadIdx.x + u * NT;
    if (i < hg * R) stf(out + ((size_t)(h0 + i / R) * T + t) * R + i % R, acc[u] * linv[i / R]);
  }
}


// ---- bf16, matrix cores: the 16 rows of a tile are 16 heads of ONE token (every head reads the same cache
// rows, so the heads are the M dimension of the products, for a decode row as for a prompt row).  A workgroup
// of 4 waves takes (token, 16 heads); wave w visits the key tiles w, w + 4, ... (16 keys, one page: the tiles
// are page-aligned) with its own online softmax:
//   scores   S[16 heads x 16 keys] on MFMA 16x16x32 bf16: A = the staged query rows [latent | rotated part]
//            from LDS, B = 16-byte loads straight from the token-major cache rows;
//   weights  fp32; exp(S - running maximum), transposed through a per-wave LDS scratch into the A layout and
//            split into two bf16 terms (hi + mid carries 16 mantissa bits), so the product with the values
//            does not round the weights to bf16;
//   values   the first R entries of the same cache rows: the key fragments already in registers are written to
//            a per-wave LDS tile entry-major, B fragments are 8-byte LDS reads; MFMA 16x16x16 bf16, fp32
//            accumulators [16 heads x R] in registers.
// The four waves' partial results are merged in LDS (common maximum, summed denominators) and written once.
typedef short s16x4 __attribute__((ext_vector_type(4)));
constexpr int KU = 6;    // key fragments requested together
constexpr int VST = 20;  // keys per value entry in a wave's staged tile (16 + padding: 8-byte aligned rows)
constexpr int PST = 20;   // row stride of the weight scratch (floats): 16-byte aligned rows, no bank conflicts on the transpose

template <int NB>
__global__ __launch_bounds__(NT) void window_attention_tile_kernel(bf16_t* __restrict__ out,
                                                                   const bf16_t* __restrict__ q_lat,
                                                                   const float* __restrict__ q_rot,
                                                                   const bf16_t* __restrict__ cache, WinArgs a) {
  extern __shared__ float lds[];
  const int R = a.R, Dr = a.Dr, E = R + Dr, H = a.H, T = a.T, BS = a.BS;
  const int QST = E + 8;                          // query row stride: 16 more bytes, so the 16 rows' fragments fall in different banks
  bf16_t* Qs = reinterpret_cast<bf16_t*>(lds);   // [16][QST]
  float* Pt = lds + 8 * QST;                      // [NW][16][PST]
  float* ML = Pt + NW * 16 * PST;                 // [NW][16][2] running (maximum, denominator) of each wave
  float* INV = ML + NW * 16 * 2;                  // [16] 1 / total denominator
  float* Acc = INV + 16;                          // [16][R] the merged result; the same memory holds, during the key
  bf16_t* vs = reinterpret_cast<bf16_t*>(Acc) + (size_t)(threadIdx.x >> 6) * R * VST;   // loop, each wave's value tile [R][VST]
  const int t = blockIdx.x, h0 = blockIdx.y * 16;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int nh = min(16, H - h0);
  if (a.slots[t] < 0) {
    for (int i = tid; i < nh * R; i += NT) out[((size_t)(h0 + i / R) * T + t) * R + i % R] = 0;
    return;
  }
  const int p = a.positions[t];
  const int* bt = a.block_tables + (size_t)seq_of(a.q_starts, a.num_seqs, t) * a.max_blocks;
  const int start = a.window > 0 ? max(0, p - a.window + 1) : 0;
  const int jt0 = start & ~15;
  {   // the 16 query rows: the latent parts in 16-byte pieces, the rotated parts converted to bf16
    const int c8 = R >> 3;
    for (int i = tid; i < 16 * c8; i += NT) {
      const int r = i / c8, c = i - r * c8, h = min(h0 + r, H - 1);
      *reinterpret_cast<uint4*>(Qs + r * QST + 8 * c) = *reinterpret_cast<const uint4*>(q_lat + ((size_t)h * T + t) * R + 8 * c);
    }
    for (int i = tid; i < 16 * Dr; i += NT) {
      const int r = i / Dr, e = i - r * Dr, h = min(h0 + r, H - 1);
      Qs[r * QST + R + e] = f2bf(q_rot[((size_t)t * H + h) * Dr + e]);
    }
  }
  __syncthreads();
  float m[4], l[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {   // the sink counts once: in wave 0
    const bool sk = a.sink != nullptr && wave == 0;
    m[r] = sk ? a.sink[min(h0 + 4 * grp + r, H - 1)] : -INFINITY;
    l[r] = sk ? 1.f : 0.f;
  }
  f32x4 pacc[NB];
#pragma unroll
  for (int db = 0; db < NB; ++db) pacc[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int nb = R >> 4, nks = E >> 5;
  const int ntiles = ((p - jt0) >> 4) + 1;
  float* pt = Pt + wave * 16 * PST;
  const bf16_t* qrow = Qs + col * QST + 8 * grp;
  for (int ti = wave; ti < ntiles; ti += NW) {
    const int jt = jt0 + 16 * ti;
    const bf16_t* base = cache + ((size_t)bt[jt / BS] * BS + (jt % BS)) * E;   // rows jt .. jt + 15 of one page
    const bf16_t* kp = base + (size_t)col * E + 8 * grp;
    // the key fragments are requested KU at a time; the first R entries of a key row are also its value, so each
    // fragment of the latent part is written to the wave's LDS tile transposed (entry-major, 16 keys side by
    // side): the B operand of weights x values is then one 8-byte LDS read
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    for (int c0 = 0; c0 < nks; c0 += KU) {
      uint4 kf[KU];
#pragma unroll
      for (int u = 0; u < KU; ++u) kf[u] = *reinterpret_cast<const uint4*>(kp + 32 * min(c0 + u, nks - 1));
#pragma unroll
      for (int u = 0; u < KU; ++u) {
        const int ks = c0 + u;
        if (ks < nks) {
          s = mfma16x16x32(as_bf16x8(*reinterpret_cast<const uint4*>(qrow + 32 * ks)), as_bf16x8(kf[u]), s);
          const int d0 = 32 * ks + 8 * grp;
          if (d0 < R) {
            bf16_t* dst = vs + (size_t)d0 * VST + col;
            const uint32_t wd[4] = {kf[u].x, kf[u].y, kf[u].z, kf[u].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              dst[(2 * i) * VST] = (bf16_t)(wd[i] & 0xffffu);
              dst[(2 * i + 1) * VST] = (bf16_t)(wd[i] >> 16);
            }
          }
        }
      }
    }
    const int jj = jt + col;
    const bool vis = jj >= start && jj <= p;
    float cr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float x = vis ? s[r] * a.scale : -INFINITY;
      const float mn = fmaxf(m[r], row16_max(x));
      float pr = 0.f, c = 1.f;
      if (mn != -INFINITY) {
        pr = vis ? __expf(x - mn) : 0.f;
        c = m[r] == -INFINITY ? 0.f : __expf(m[r] - mn);
      }
      l[r] = l[r] * c + row16_sum(pr);
      m[r] = mn;
      pt[(4 * grp + r) * PST + col] = pr;
      cr[r] = c;
    }
    if (__any(cr[0] != 1.f || cr[1] != 1.f || cr[2] != 1.f || cr[3] != 1.f)) {   // a maximum moved (rare after the first tiles)
#pragma unroll
      for (int db = 0; db < NB; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r) pacc[db][r] *= cr[r];
    }
    const f32x4 pa = *reinterpret_cast<const f32x4*>(pt + col * PST + 4 * grp);   // head `col`, keys 4 grp .. + 4
    s16x4 ahi, amid;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bf16_t hi = f2bf(pa[i]);
      ahi[i] = (short)hi;
      amid[i] = (short)f2bf(pa[i] - bf2f(hi));
    }
    const bf16_t* vrd = vs + (size_t)col * VST + 4 * grp;   // entry 16 db + col, keys 4 grp .. + 4
#pragma unroll
    for (int db = 0; db < NB; ++db) {
      if (db < nb) {
        const s16x4 b = *reinterpret_cast<const s16x4*>(vrd + (size_t)16 * db * VST);
        pacc[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ahi, b, pacc[db], 0, 0, 0);
        pacc[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(amid, b, pacc[db], 0, 0, 0);
      }
    }
  }
  // ---- merge the waves ----
  __syncthreads();   // every wave is done with its value tile: the memory becomes the merged result
  if (col == 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      ML[(wave * 16 + 4 * grp + r) * 2] = m[r];
      ML[(wave * 16 + 4 * grp + r) * 2 + 1] = l[r];
    }
  }
  __syncthreads();
  float f[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = 4 * grp + r;
    float mg = -INFINITY;
    for (int w = 0; w < NW; ++w) mg = fmaxf(mg, ML[(w * 16 + row) * 2]);
    float lt = 0.f;
    for (int w = 0; w < NW; ++w) {
      const float mw = ML[(w * 16 + row) * 2];
      if (mw != -INFINITY) lt += ML[(w * 16 + row) * 2 + 1] * __expf(mw - mg);
    }
    f[r] = m[r] == -INFINITY ? 0.f : __expf(m[r] - mg);
    if (wave == 0 && col == 0) INV[row] = 1.0f / lt;
  }
  for (int w = 0; w < NW; ++w) {
    if (wave == w) {
#pragma unroll
      for (int db = 0; db < NB; ++db) {
        if (db < nb) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int idx = (4 * grp + r) * R + 16 * db + col;
            const float v = pacc[db][r] * f[r];
            Acc[idx] = w == 0 ? v : Acc[idx] + v;
          }
        }
      }
    }
    __syncthreads();
  }
  {
    const int c4 = R >> 2;   // four results per thread and store
    for (int i = tid; i < nh * c4; i += NT) {
      const int row = i / c4, c = i - row * c4;
      const f32x4 v = *reinterpret_cast<const f32x4*>(Acc + row * R + 4 * c);
      const float inv = INV[row];
      uint2 pk = {pack2(v[0] * inv, v[1] * inv), pack2(v[2] * inv, v[3] * inv)};
      *reinterpret_cast<uint2*>(out + ((size_t)(h0 + row) * T + t) * R + 4 * c) = pk;
    }
  }
}

template <int NB>
int launch_tile(bf16_t* out, const bf16_t* q_lat, const float* q_rot, const bf16_t* cache, const WinArgs& a,
                hipStream_t st) {
  const int E = a.R + a.Dr;
  // the value tiles (NW x R x VST bf16) and the merged result (16 x R fp32) share memory
  const size_t tail = (size_t)a.R * (NW * VST * 2 > 16 * 4 ? NW * VST * 2 : 16 * 4);
  const size_t lds = (size_t)(8 * (E + 8) + NW * 16 * PST + NW * 16 * 2 + 16) * sizeof(float) + tail;
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(window_attention_tile_kernel<NB>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  dim3 grid(a.T, (a.H + 15) / 16);
  window_attention_tile_kernel<NB><<<grid, NT, lds, st>>>(out, q_lat, q_rot, cache, a);
  KA_CHECK_LAUNCH();
}

}  // namespace

extern "C" int ka_latent_prep(void* cq, const void* proj, int T, int P, int Q, int R, int Dr, const float* w_q,
                              const float* w_kv, const float* inv_freq, const int* positions, const int* slots,
                              void* cache, int rot_dims, float eps, int interleaved, float mag, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (Q < 0 || P < Q || (Q == 0 && cache == nullptr) || (cache != nullptr && (P < Q + R + Dr || R <= 0)) || rot_dims < 0 || rot_dims > Dr || (rot_dims & 1))
    return (int)hipErrorInvalidValue;
  if (f32)
    latent_prep_kernel<float><<<T, NT, 0, st>>>((float*)cq, (const float*)proj, P, Q, R, Dr, w_q, w_kv, inv_freq, positions,
                                                slots, (float*)cache, rot_dims, eps, interleaved, mag);
  else
    latent_prep_kernel<bf16_t><<<T, NT, 0, st>>>((bf16_t*)cq, (const bf16_t*)proj, P, Q, R, Dr, w_q, w_kv, inv_freq,
                                                 positions, slots, (bf16_t*)cache, rot_dims, eps, interleaved, mag);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_rope_split_q(void* qn, float* qr, const void* q, int P, int off, const float* inv_freq,
                               const int* positions, int T, int H, int D, int Dr, int rot_dims, int interleaved, float mag,
                               int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (rot_dims < 0 || rot_dims > Dr || (rot_dims & 1) || off < 0 || off + H * (D + Dr) > P) return (int)hipErrorInvalidValue;
  if (f32)
    rope_split_q_kernel<float><<<T, NT, 0, st>>>((float*)qn, qr, (const float*)q, P, off, inv_freq, positions, T, H, D, Dr,
                                                 rot_dims, interleaved, mag);
  else
    rope_split_q_kernel<bf16_t><<<T, NT, 0, st>>>((bf16_t*)qn, qr, (const bf16_t*)q, P, off, inv_freq, positions, T, H, D, Dr,
                                                  rot_dims, interleaved, mag);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_head_gate(void* out, const void* o, const void* gate, int gs, int g_off, int T, int H, int Dv, int f32,
                            hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || Dv <= 0 || (gate != nullptr && (g_off < 0 || g_off + H > gs))) return (int)hipErrorInvalidValue;
  if (f32) head_gate_kernel<float><<<T, NT, 0, st>>>((float*)out, (const float*)o, (const float*)gate, gs, g_off, T, H, Dv);
  else head_gate_kernel<bf16_t><<<T, NT, 0, st>>>((bf16_t*)out, (const bf16_t*)o, (const bf16_t*)gate, gs, g_off, T, H, Dv);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_window_attention(void* out, const void* q_lat, const float* q_rot, const void* cache,
                                   const int* block_tables, const int* q_starts, int num_seqs, const int* positions,
                                   const int* slots, const float* sink, int T, int H, int R, int Dr, int BS,
                                   int max_blocks, int window, float scale, int f32, int mode, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || R <= 0 || Dr < 0 || BS <= 0 || window < 0 || R > NT * MAX_ACC) return (int)hipErrorInvalidValue;
  if (!f32 && mode == 0 && R % 16 == 0 && R <= 512 && (R + Dr) % 32 == 0 && BS % 16 == 0) {   // the matrix-core kernel
    WinArgs a{block_tables, q_starts, num_seqs, positions, slots, sink, T, H, 16, R, Dr, BS, max_blocks, window, scale};
    const int nb = R / 16;
    bf16_t* o = (bf16_t*)out;
    const bf16_t* ql = (const bf16_t*)q_lat;
    const bf16_t* kc = (const bf16_t*)cache;
    if (nb <= 4) return launch_tile<4>(o, ql, q_rot, kc, a, st);
    if (nb <= 8) return launch_tile<8>(o, ql, q_rot, kc, a, st);
    if (nb <= 16) return launch_tile<16>(o, ql, q_rot, kc, a, st);
    return launch_tile<32>(o, ql, q_rot, kc, a, st);
  }
  // heads per workgroup: as many as the accumulators (NT * MAX_ACC outputs), the 16 running values per wave
  // and 120 KB of LDS allow
  int HG = min(H, min(NT * MAX_ACC / R, 16 * NW));
  while (HG > 1 && (size_t)(HG * (R + Dr + KT + 2)) * sizeof(float) > 120 * 1024) --HG;
  const size_t lds = (size_t)(HG * (R + Dr + KT + 2)) * sizeof(float);
  if (lds > 120 * 1024) return (int)hipErrorInvalidValue;
  WinArgs a{block_tables, q_starts, num_seqs, positions, slots, sink, T, H, HG, R, Dr, BS, max_blocks, window, scale};
  const void* fn = f32 ? reinterpret_cast<const void*>(window_attention_kernel<float>)
                       : reinterpret_cast<const void*>(window_attention_kernel<bf16_t>);
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  dim3 grid(T, (H + HG - 1) / HG);
  if (f32)
    window_attention_kernel<float><<<grid, NT, lds, st>>>((float*)out, (const float*)q_lat, q_rot, (const float*)cache, a);
  else
    window_attention_kernel<bf16_t><<<grid, NT, lds, st>>>((bf16_t*)out, (const bf16_t*)q_lat, q_rot, (const bf16_t*)cache, a);
  KA_CHECK_LAUNCH();
}
