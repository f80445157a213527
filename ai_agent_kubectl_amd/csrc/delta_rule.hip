// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// The gated delta rule: a recurrent mixer with a matrix memory S [D, Dv] per head (models/suvapel.py).  Per head
// and row, with unit vectors q, k [D] (q also scaled by D^-1/2), the value v [Dv], a write strength beta in (0, 1)
// and a decay g in (0, 1), one number per head or one per key channel:
//
//   S <- g * S                     (per channel: row d of S times g[d])
//   u  = beta * (v - S^T k)        what the memory returns for k is replaced by v, as far as beta says
//   S <- S + k u^T
//   o  = S^T q                     read after the write: o contains beta (v - S^T k) (k . q)
//
// All of it is fp32.  `delta_prep` makes the fp32 inputs from the convolved projection rows (unit norms, sigmoid,
// softplus, the two exponentials of the decay).  `delta_scan` runs the recurrence over the rows that each sequence
// brings to this step, from the memory in the sequence's state slot and back into it; a sequence whose first row is
// at position 0 starts from the zero memory, so a slot needs no clearing between requests.  The same launch serves
// a decode step (one row per sequence) and a prompt portion of any length; a row's arithmetic does not depend on
// how the rows were cut into steps.
//
// A column S[:, c] evolves on its own given the row's k, q, g, beta and v[c], so a column is held by DPL adjacent
// lanes, each with RPT consecutive entries in registers; q, k (and g) rows come from LDS as broadcast 16-byte
// pieces.  Both read-outs of the decayed memory, S^T k and S^T q, are reduced side by side, and the row's own write
// enters the result as u[c] * (k . q):  (S + k u^T)^T q = S^T q + u (k . q).
#include "rows_f32.h"

namespace {
using namespace rows;

constexpr int MAX_DL = 8;   // head entries per lane in delta_prep: D <= 64 * MAX_DL

template <typename AT>
__global__ __launch_bounds__(NT) void delta_prep_kernel(float* __restrict__ qk, float* __restrict__ beta,
                                                        float* __restrict__ decay, const AT* __restrict__ cv, int cs,
                                                        const AT* __restrict__ beta_src, int bs, int b_off,
                                                        const AT* __restrict__ a_src, int as, int a_off,
                                                        const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                        int H, int G, int D, int channel) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float qscale = 1.0f / sqrtf((float)D);
  for (int hh = wave; hh < 2 * G; hh += NW) {           // q heads 0 .. G - 1, then k heads
    const AT* x = cv + (size_t)t * cs + (size_t)hh * D;
    float v[MAX_DL];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < MAX_DL; ++u) {
      const int i = lane + 64 * u;
      v[u] = i < D ? ldf(x + i) : 0.f;
      ss += v[u] * v[u];
    }
    const float inv = (1.0f / sqrtf(wave_sum(ss) + 1e-6f)) * (hh < G ? qscale : 1.0f);
    float* dst = qk + ((size_t)t * 2 * G + hh) * D;
#pragma unroll
    for (int u = 0; u < MAX_DL; ++u) {
      const int i = lane + 64 * u;
      if (i < D) dst[i] = v[u] * inv;
    }
  }
  for (int h = threadIdx.x; h < H; h += NT)
    beta[(size_t)t * H + h] = 1.0f / (1.0f + expf(-ldf(beta_src + (size_t)t * bs + b_off + h)));
  const int n = channel ? H * D : H;
  for (int i = threadIdx.x; i < n; i += NT) {
    const float a = ldf(a_src + (size_t)t * as + a_off + i) + dt_bias[i];
    const float sp = a > 20.f ? a : log1pf(expf(a));                 // softplus
    decay[(size_t)t * n + i] = expf(-expf(A_log[channel ? i / D : i]) * sp);
  }
}

struct ScanArgs {
  const int* q_starts;     // [num_seqs + 1] or null (row t is sequence t)
  const int* seq_slots;    // [num_seqs] state slot, < 0: skip
  const int* positions;    // [T]
  int vs, v_off;           // value row stride and column offset
  int H, G, D, Dv;
  int channel;             // decay [T, H, D] instead of [T, H]
};

template <int DPL>
KA_DEV float col_sum(float v) {
  if constexpr (DPL == 4) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    return v;
  } else if constexpr (DPL == 8) {
    v += dpp_f<0xB1>(v);
    v += dpp_f<0x4E>(v);
    v += dpp_f<0x141>(v);
    return v;
  } else {
    return row16_sum(v);
  }
}

// S [slots, H, Dv, D]: a column's D entries are contiguous.  A workgroup takes (sequence, head, NT / DPL columns).
template <typename AT, int RPT, int DPL>
__global__ __launch_bounds__(NT) void delta_scan_kernel(float* __restrict__ out, const float* __restrict__ qk,
                                                        const AT* __restrict__ v_src, const float* __restrict__ beta,
                                                        const float* __restrict__ decay, float* __restrict__ st_S,
                                                        ScanArgs a, int TB) {
  extern __shared__ float lds[];
  constexpr int Dp = DPL * RPT, CW = NT / DPL;   // D padded; columns per workgroup
  float* qs = lds;                      // [TB][Dp]
  float* ks = qs + TB * Dp;             // [TB][Dp]
  float* vs = ks + TB * Dp;             // [TB][CW]
  float* bt = vs + TB * CW;             // [TB] beta
  float* kq = bt + TB;                  // [TB] k . q
  float* gs = kq + TB;                  // [TB] (one decay per head) or [TB][Dp] (one per key channel)
  // workgroups are numbered sequence by sequence, the step's last sequence first: a mixed step lists its one-row
  // sequences first and its prompt portions last, and the long-running workgroups of the portions, dispatched first
  // and in a row, spread evenly over the CUs (interleaved with one-row workgroups they pile up on a part of them)
  const int H = a.H, G = a.G, D = a.D, Dv = a.Dv;
  const int seq = gridDim.y - 1 - blockIdx.y, h = blockIdx.x % H, zb = blockIdx.x / H;
  const int slot = a.seq_slots[seq];
  if (slot < 0) return;
  const int r0 = a.q_starts ? a.q_starts[seq] : seq, r1 = a.q_starts ? a.q_starts[seq + 1] : seq + 1;
  if (r1 <= r0) return;
  const int g = h / (H / G);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = threadIdx.x / DPL, dp = threadIdx.x % DPL;
  const int c = zb * CW + col;
  const bool cok = c < Dv;
  float* Sp = st_S + (((size_t)slot * H + h) * Dv + (cok ? c : 0)) * D;
  const bool fresh = a.positions[r0] == 0;
  const bool whole = cok && (dp + 1) * RPT <= D && (D & 3) == 0;   // this lane's entries in aligned 16-byte pieces
  float S[RPT];
#pragma unroll
  for (int u = 0; u < RPT / 4; ++u) {
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
    if (!fresh) {
      if (whole) {
        x = *reinterpret_cast<const f32x4*>(Sp + dp * RPT + 4 * u);
      } else if (cok) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (dp * RPT + 4 * u + i < D) x[i] = Sp[dp * RPT + 4 * u + i];
      }
    }
    S[4 * u] = x[0];
    S[4 * u + 1] = x[1];
    S[4 * u + 2] = x[2];
    S[4 * u + 3] = x[3];
  }
  // pad entries (d >= D) of q and k stay zero, of a per-channel decay one: a padded memory entry stays zero
  if (Dp != D) {
    for (int idx = threadIdx.x; idx < 2 * TB * Dp; idx += NT) qs[idx] = 0.f;
    if (a.channel)
      for (int idx = threadIdx.x; idx < TB * Dp; idx += NT) gs[idx] = 1.f;
  }
  const int c0 = zb * CW;
  for (int t0 = r0; t0 < r1; t0 += TB) {
    const int nt = min(TB, r1 - t0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < nt * D; idx += NT) {
      const int tt = idx / D, d = idx % D;
      const float* row = qk + ((size_t)(t0 + tt) * 2 * G + g) * D + d;
      qs[tt * Dp + d] = row[0];
      ks[tt * Dp + d] = row[(size_t)G * D];
      if (a.channel) gs[tt * Dp + d] = decay[((size_t)(t0 + tt) * H + h) * D + d];
    }
    for (int idx = threadIdx.x; idx < nt * CW; idx += NT) {
      const int tt = idx / CW, cc = c0 + idx % CW;
      vs[idx] = cc < Dv ? ldf(v_src + (size_t)(t0 + tt) * a.vs + a.v_off + h * Dv + cc) : 0.f;
    }
    for (int tt = threadIdx.x; tt < nt; tt += NT) {
      bt[tt] = beta[(size_t)(t0 + tt) * H + h];
      if (!a.channel) gs[tt] = decay[(size_t)(t0 + tt) * H + h];
    }
    __syncthreads();
    for (int tt = wave; tt < nt; tt += NW) {          // k . q of each staged row, one wave a row
      float s = 0.f;
      for (int d = lane; d < D; d += 64) s += ks[tt * Dp + d] * qs[tt * Dp + d];
      s = wave_sum(s);
      if (lane == 0) kq[tt] = s;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const f32x4* k4 = reinterpret_cast<const f32x4*>(ks + tt * Dp + dp * RPT);
      const f32x4* q4 = reinterpret_cast<const f32x4*>(qs + tt * Dp + dp * RPT);
      const f32x4* g4 = reinterpret_cast<const f32x4*>(gs + tt * Dp + dp * RPT);
      const float gh = a.channel ? 1.f : gs[tt];
      float pk0 = 0.f, pk1 = 0.f, pq0 = 0.f, pq1 = 0.f;
#pragma unroll
      for (int u = 0; u < RPT / 4; ++u) {
        const f32x4 kc = k4[u], qc = q4[u];
        f32x4 gc = {gh, gh, gh, gh};
        if (a.channel) gc = g4[u];
#pragma unroll
        for (int i = 0; i < 4; ++i) S[4 * u + i] *= gc[i];
        pk0 += S[4 * u] * kc[0] + S[4 * u + 2] * kc[2];
        pk1 += S[4 * u + 1] * kc[1] + S[4 * u + 3] * kc[3];
        pq0 += S[4 * u] * qc[0] + S[4 * u + 2] * qc[2];
        pq1 += S[4 * u + 1] * qc[1] + S[4 * u + 3] * qc[3];
      }
      const float pk = col_sum<DPL>(pk0 + pk1), pq = col_sum<DPL>(pq0 + pq1);
      const float uu = bt[tt] * (vs[tt * CW + col] - pk);
#pragma unroll
      for (int u = 0; u < RPT / 4; ++u) {
        const f32x4 kc = k4[u];
#pragma unroll
        for (int i = 0; i < 4; ++i) S[4 * u + i] += kc[i] * uu;
      }
      if (dp == 0 && cok) out[((size_t)(t0 + tt) * H + h) * Dv + c] = pq + uu * kq[tt];
    }
  }
  if (whole) {
#pragma unroll
    for (int u = 0; u < RPT / 4; ++u)
      *reinterpret_cast<f32x4*>(Sp + dp * RPT + 4 * u) = f32x4{S[4 * u], S[4 * u + 1], S[4 * u + 2], S[4 * u + 3]};
  } else if (cok) {
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
      const int d = dp * RPT + r;
      if (d < D) Sp[d] = S[r];
    }
  }
}

template <typename AT, int RPT, int DPL>
int launch_scan(float* out, const float* qk, const AT* v_src, const float* beta, const float* decay, float* S, ScanArgs a,
                int num_seqs, hipStream_t st) {
  constexpr int Dp = RPT * DPL, CW = NT / DPL;
  int TB = 4096 / Dp;   // rows staged per tile
  TB = TB < 8 ? 8 : (TB > 64 ? 64 : TB);
  const size_t lds = (size_t)(2 * TB * Dp + TB * CW + 2 * TB + (a.channel ? TB * Dp : TB)) * sizeof(float);
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(delta_scan_kernel<AT, RPT, DPL>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  if (num_seqs > 65535) return (int)hipErrorInvalidValue;
  dim3 grid(a.H * ((a.Dv + CW - 1) / CW), num_seqs);
  delta_scan_kernel<AT, RPT, DPL><<<grid, NT, lds, st>>>(out, qk, v_src, beta, decay, S, a, TB);
  KA_CHECK_LAUNCH();
}

// lanes per column: 0 = by the head size; 4, 8 or 16 = that many (more lanes: shorter chains per row and more
// workgroups, at the price of staging the q / k rows once per narrower block of columns)
template <typename AT>
int dispatch_scan(float* out, const float* qk, const AT* v_src, const float* beta, const float* decay, float* S,
                  const ScanArgs& a, int num_seqs, int lanes, hipStream_t st) {
  const int D = a.D;
  // few workgroups (a step with few sequences): eight lanes a column double them and halve a row's chain
  if (lanes == 0 && D > 32 && D <= 128 && (long)num_seqs * a.H * ((a.Dv + 63) / 64) <= 256) lanes = 8;
#define KA_S(RPT, DPL) return launch_scan<AT, RPT, DPL>(out, qk, v_src, beta, decay, S, a, num_seqs, st)
  if (D <= 16) KA_S(4, 4);
  if (D <= 32) {
    if (lanes == 8) KA_S(4, 8);
    KA_S(8, 4);
  }
  if (D <= 64) {
    if (lanes == 16) KA_S(4, 16);
    if (lanes == 8) KA_S(8, 8);
    KA_S(16, 4);
  }
  if (D <= 128) {
    if (lanes == 16) KA_S(8, 16);
    if (lanes == 8) KA_S(16, 8);
    KA_S(32, 4);
  }
  if (D <= 256) {
    if (lanes == 4) KA_S(64, 4);
    if (lanes == 8) KA_S(32, 8);
    KA_S(16, 16);
  }
  KA_S(32, 16);
#undef KA_S
}

}  // namespace

extern "C" int ka_delta_prep(float* qk, float* beta, float* decay, const void* cv, int cs, const void* beta_src, int bs,
                             int b_off, const void* a_src, int as, int a_off, const float* A_log, const float* dt_bias,
                             int T, int H, int G, int D, int channel, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || D > 64 * MAX_DL || 2 * G * D > cs || b_off < 0 || b_off + H > bs ||
      a_off < 0 || a_off + (channel ? H * D : H) > as)
    return (int)hipErrorInvalidValue;
  if (f32)
    delta_prep_kernel<float><<<T, NT, 0, st>>>(qk, beta, decay, (const float*)cv, cs, (const float*)beta_src, bs, b_off,
                                               (const float*)a_src, as, a_off, A_log, dt_bias, H, G, D, channel);
  else
    delta_prep_kernel<bf16_t><<<T, NT, 0, st>>>(qk, beta, decay, (const bf16_t*)cv, cs, (const bf16_t*)beta_src, bs, b_off,
                                                (const bf16_t*)a_src, as, a_off, A_log, dt_bias, H, G, D, channel);
  KA_CHECK_LAUNCH();
}

// out [T, H * Dv] fp32 (rows of no sequence are left as they are)
extern "C" int ka_delta_scan(float* out, const float* qk, const void* v_src, int vs, int v_off, const float* beta,
                             const float* decay, float* st_S, const int* seq_slots, const int* q_starts, int num_seqs,
                             const int* positions, int H, int G, int D, int Dv, int channel, int lanes, int f32,
                             hipStream_t st) {
  if (num_seqs <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || D <= 0 || D > 512 || Dv <= 0 || H > 65535 || v_off < 0 || v_off + H * Dv > vs)
    return (int)hipErrorInvalidValue;
  ScanArgs a{q_starts, seq_slots, positions, vs, v_off, H, G, D, Dv, channel};
  if (f32) return dispatch_scan<float>(out, qk, (const float*)v_src, beta, decay, st_S, a, num_seqs, lanes, st);
  return dispatch_scan<bf16_t>(out, qk, (const bf16_t*)v_src, beta, decay, st_S, a, num_seqs, lanes, st);
}
