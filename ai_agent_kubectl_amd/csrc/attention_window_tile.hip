// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Sliding-window attention with kept first tokens on the matrix cores (bf16 prompt portions; the mask, the gate and
// the cache layout are those of attention_window.hip).
//
// One workgroup per (sequence, 16 consecutive query rows, key/value head); its H / G waves are the query heads that
// share the key/value head, so they read the same pages at about the same time.  A wave walks the pages that any of
// its rows can see (the kept first pages, then the pages of the rows' windows), four pages = 64 keys per step:
//   scores, transposed:  S^T[key][query] = K Q^T on MFMA 16x16x32 bf16.  A = a page's 16 keys (16-byte loads straight
//       from the token-major page), B = the wave's query rows (resident).  A lane then holds, for ONE query
//       (lane & 15), the scores of four consecutive keys (4 (lane >> 4) + r): the layout of the next product's A operand.
//   softmax online in fp32 per query: the step's maximum over the lane's 16 scores and two lane swaps; the running sum
//       stays a per-lane partial (the rescale factor is the same in the four lanes of a query) and is summed at the end.
//   weights x values:  O[query][entry] += P V on MFMA 16x16x16 bf16 with every fp32 weight split into two bf16 terms
//       (hi + lo carries 16 mantissa bits), A = the weights as they lie in the registers, B = 8-byte loads from the
//       entry-major value page (4 consecutive keys of one entry).
// No LDS, no barrier.  The rescale factors and the final 1 / sum * sigmoid(gate) reach the accumulator rows (queries
// 4 (lane >> 4) + r) by lane reads.  Slots of the last page beyond the rows' positions may hold another sequence's
// old values: their weights are zero and their value bits are cleared before the product.
// SIG (SlideArgs::dist set): the weights are sigmoids of the biased scores and final as they are, so the maximum, the
// rescale and the denominator fall away and the waves' partial results of a single row are simply added.
#include "attention_window.h"

typedef short s16x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int PG = 16;   // page size = keys per MFMA tile
constexpr int NP = 4;    // pages per softmax step

KA_DEV void split2(const f32x4& p, s16x4& hi, s16x4& lo) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bf16_t h = f2bf(p[i]);
    hi[i] = (short)h;
    lo[i] = (short)f2bf(p[i] - bf2f(h));
  }
}

// DEC false: a prompt portion.  The 16 query columns of a wave are 16 consecutive rows of one sequence for one query
//   head; the workgroup's waves are the heads of the key/value group.
// DEC true: single rows (a decode step, or the one-row sequences of a mixed step).  The query columns are the H / G
//   heads of the key/value group for ONE row, so a page is read once for all of them; the workgroup's four waves
//   take every fourth step of the pages with a softmax of their own and are merged through LDS at the end.
template <int DK, int DB, bool DEC, bool SIG>   // D = 32 DK, Dv = 16 DB
__global__ __launch_bounds__(512) void sliding_tile_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ q,
                                                           const bf16_t* __restrict__ k_cache,
                                                           const bf16_t* __restrict__ v_cache,
                                                           const bf16_t* __restrict__ gate, SlideArgs a, int tiles_per_seq) {
  constexpr int D = 32 * DK, Dv = 16 * DB;
  extern __shared__ float lds[];   // DEC: [nw][rep] maxima, [nw][rep] sums, [nw][rep][Dv] partial results
  const int g = blockIdx.y, H = a.H, G = a.G, rep = H / G;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  int seq, r0, nq, P0, p_last;
  if constexpr (DEC) {
    seq = r0 = blockIdx.x;                         // row t is block-table row t
    nq = rep;
    if (a.slots[r0] < 0) {                         // a padding row
      for (int i = threadIdx.x; i < rep * Dv; i += blockDim.x) out[((size_t)r0 * H + g * rep) * Dv + i] = 0;
      return;
    }
    P0 = p_last = a.positions[r0];
  } else {
    seq = blockIdx.x / tiles_per_seq;
    r0 = a.q_starts[seq] + (blockIdx.x % tiles_per_seq) * 16;
    const int r1 = a.q_starts[seq + 1];
    if (r0 >= r1) return;
    nq = min(16, r1 - r0);
    P0 = a.positions[r0];                          // the rows' positions are P0, P0 + 1, ...
    p_last = P0 + nq - 1;
  }
  const int* bt = a.block_tables + (size_t)seq * a.max_blocks;
  const int W = a.window > 0 ? a.window : 0x3fffffff;
  const bool valid_q = col < nq;
  const int cq = min(col, nq - 1);
  const int p_q = DEC ? P0 : P0 + col;             // this lane's query position
  const int row_q = DEC ? r0 : r0 + cq;            // its row of q / gate / out
  const int h_q = g * rep + (DEC ? cq : wave);     // its query head
  float r1 = 0.f, r2 = 0.f, pb = 0.f;              // the lane's head's distance bias and score offset
  if constexpr (SIG) {
    r1 = a.dist[h_q];
    r2 = a.dist[H + h_q];
    pb = a.dist[2 * H + h_q];
  }
  bf16x8 qf[DK];
  {
    const bf16_t* qp = q + ((size_t)row_q * H + h_q) * D + 8 * grp;
#pragma unroll
    for (int kk = 0; kk < DK; ++kk) qf[kk] = as_bf16x8(*reinterpret_cast<const uint4*>(qp + 32 * kk));
  }
  // pages: the kept first ones that lie before the first window page, then the window pages of all rows
  const int first_w = max(0, P0 - W + 1) / PG, last_pg = p_last / PG;
  const int keep_end = min(a.keep_first, max(0, p_last - W + 1));
  const int nkp = min((keep_end + PG - 1) / PG, first_w);
  const int total = nkp + (last_pg - first_w + 1);
  float m_run = -INFINITY, l_run = 0.f;
  f32x4 O[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) O[db] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int i0 = DEC ? wave * NP : 0; i0 < total; i0 += DEC ? nw * NP : NP) {
    f32x4 sv[NP];
    int pbase[NP], pgs[NP];
    float mt = -INFINITY;
#pragma unroll
    for (int u = 0; u < NP; ++u) {
      const int i = i0 + u;
      sv[u] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      pbase[u] = 0;
      pgs[u] = 0;
      if (i < total) {                            // wave-uniform
        const int pg = i < nkp ? i : first_w + (i - nkp);
        pgs[u] = pg;
        pbase[u] = bt[pg] * G + g;
        const bf16_t* kp = k_cache + ((size_t)pbase[u] * PG + col) * D + 8 * grp;
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < DK; ++kk) s = mfma16x16x32(as_bf16x8(*reinterpret_cast<const uint4*>(kp + 32 * kk)), qf[kk], s);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int j = pg * PG + 4 * grp + r;
          const bool ok = valid_q && j <= p_q && (p_q - j < W || j < a.keep_first);
          if constexpr (SIG) {
            const float z = s[r] * a.scale - r1 * __logf(1.0f + r2 * (float)(p_q - j)) + pb;
            sv[u][r] = ok ? 1.0f / (1.0f + __expf(-z)) : 0.f;
          } else {
            sv[u][r] = ok ? s[r] * a.scale : -INFINITY;
            mt = fmaxf(mt, sv[u][r]);
          }
        }
      } else if constexpr (SIG) {
        sv[u] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
    }
    if constexpr (!SIG) {
      mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
      mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
      const float m_new = fmaxf(m_run, mt);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;          // a query that has seen no key yet
      const float corr = m_run == -INFINITY ? 1.f : __expf(m_run - m_use);
      m_run = m_new;
      float psum = 0.f;
#pragma unroll
      for (int u = 0; u < NP; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float e = sv[u][r] == -INFINITY ? 0.f : __expf(sv[u][r] - m_use);
          sv[u][r] = e;
          psum += e;
        }
      l_run = l_run * corr + psum;
      if (!__all(corr == 1.f)) {
        float cr[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) cr[r] = __shfl(corr, 4 * grp + r, 64);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r) O[db][r] *= cr[r];
      }
    }
#pragma unroll
    for (int u = 0; u < NP; ++u) {
      if (i0 + u < total) {
        s16x4 ahi, alo;
        split2(sv[u], ahi, alo);
        const bf16_t* vp = v_cache + ((size_t)pbase[u] * Dv + col) * PG + 4 * grp;
        const int over = pgs[u] * PG + 4 * grp + 3 - p_last;       // > 0: this lane's last `over` keys lie beyond the rows
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          s16x4 b = *reinterpret_cast<const s16x4*>(vp + (size_t)16 * db * PG);
          if (over > 0) {
#pragma unroll
            for (int k = 0; k < 4; ++k)
              if (3 - k < over) b[k] = 0;
          }
          O[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ahi, b, O[db], 0, 0, 0);
          O[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(alo, b, O[db], 0, 0, 0);
        }
      }
    }
  }
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  if constexpr (DEC) {
    // merge the waves' partial softmaxes: out = sum_w O_w e^(m_w - M) / sum_w l_w e^(m_w - M)
    float* sm = lds;                     // [nw][rep]
    float* sl = sm + nw * rep;           // [nw][rep]
    float* so = sl + nw * rep;           // [nw][rep][Dv]
    if (grp == 0 && col < rep) {   // SIG: equal maxima and denominators 1 / nw make the merge below a plain sum
      sm[wave * rep + col] = SIG ? 0.f : m_run;
      sl[wave * rep + col] = SIG ? 1.0f / (float)nw : l_run;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int hq = 4 * grp + r;
      if (hq < rep) {
#pragma unroll
        for (int db = 0; db < DB; ++db) so[((size_t)wave * rep + hq) * Dv + 16 * db + col] = O[db][r];
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < rep * Dv; i += blockDim.x) {
      const int hq = i / Dv, d = i % Dv;
      float M = -INFINITY;
      for (int w = 0; w < nw; ++w) M = fmaxf(M, sm[w * rep + hq]);
      float num = 0.f, den = 0.f;
      for (int w = 0; w < nw; ++w) {
        const float mw = sm[w * rep + hq];
        const float f = mw == -INFINITY ? 0.f : __expf(mw - M);
        num += so[((size_t)w * rep + hq) * Dv + d] * f;
        den += sl[w * rep + hq] * f;
      }
      float o = num / den;
      if (gate != nullptr) o *= 1.0f / (1.0f + __expf(-bf2f(gate[(size_t)r0 * a.gs + a.g_off + g * rep + hq])));
      out[((size_t)r0 * H + g * rep + hq) * Dv + d] = f2bf(o);
    }
  } else {
    float fin = valid_q ? (SIG ? 1.0f : 1.0f / l_run) : 0.f;
    if (gate != nullptr && valid_q) fin *= 1.0f / (1.0f + __expf(-bf2f(gate[(size_t)row_q * a.gs + a.g_off + h_q])));
    float fr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) fr[r] = __shfl(fin, 4 * grp + r, 64);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * grp + r;
      if (row < nq) {
        bf16_t* op = out + ((size_t)(r0 + row) * H + h_q) * Dv + col;
#pragma unroll
        for (int db = 0; db < DB; ++db) op[16 * db] = f2bf(O[db][r] * fr[r]);
      }
    }
  }
}

constexpr int DEC_WAVES = 4;

template <int DK, int DB, bool SIG>
int launch_tile(bf16_t* out, const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const bf16_t* gate,
                const SlideArgs& a, int max_q, int rows_, hipStream_t st) {
  if (a.q_starts == nullptr) {   // single rows
    const int rep = a.H / a.G;
    const size_t lds = (size_t)(DEC_WAVES * rep * (2 + 16 * DB)) * sizeof(float);
    if (lds > 64 * 1024) return (int)hipErrorInvalidValue;
    if (lds > 48 * 1024) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(sliding_tile_kernel<DK, DB, true, SIG>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return (int)e;
    }
    sliding_tile_kernel<DK, DB, true, SIG><<<dim3(rows_, a.G), 64 * DEC_WAVES, lds, st>>>(out, q, k_cache, v_cache, gate, a, 1);
  } else {
    const int tiles = (max_q + 15) / 16;
    sliding_tile_kernel<DK, DB, false, SIG><<<dim3(a.num_seqs * tiles, a.G), 64 * (a.H / a.G), 0, st>>>(out, q, k_cache, v_cache,
                                                                                                 gate, a, tiles);
  }
  KA_CHECK_LAUNCH();
}

}  // namespace

extern "C" int ka_sliding_attention_tile_ok(int H, int G, int D, int Dv, int BS) {
  return BS == PG && G > 0 && H % G == 0 && H / G <= 8 && (D == 64 || D == 128 || D == 256) &&
         (Dv == 64 || Dv == 128 || Dv == 256);
}

// q_starts set: a varlen step, `max_q` its longest run of rows; rows of no sequence (padding after the last one) are
// not written: the caller clears `out`.  q_starts null: `rows_` single rows, row t is block-table row t.
int sliding_attention_tile(bf16_t* out, const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const bf16_t* gate,
                           const SlideArgs& a, int max_q, int rows_, hipStream_t st) {
  if (!ka_sliding_attention_tile_ok(a.H, a.G, a.D, a.Dv, a.BS) || (a.q_starts != nullptr ? max_q <= 0 : rows_ <= 0))
    return (int)hipErrorInvalidValue;
#define KA_T(DK, DB)                                                                                        \
  return a.dist != nullptr ? launch_tile<DK, DB, true>(out, q, k_cache, v_cache, gate, a, max_q, rows_, st) \
                           : launch_tile<DK, DB, false>(out, q, k_cache, v_cache, gate, a, max_q, rows_, st)
  if (a.D == 64) {
    if (a.Dv == 64) KA_T(2, 4);
    if (a.Dv == 128) KA_T(2, 8);
    KA_T(2, 16);
  }
  if (a.D == 128) {
    if (a.Dv == 64) KA_T(4, 4);
    if (a.Dv == 128) KA_T(4, 8);
    KA_T(4, 16);
  }
  if (a.Dv == 64) KA_T(8, 4);
  if (a.Dv == 128) KA_T(8, 8);
  KA_T(8, 16);
#undef KA_T
}
