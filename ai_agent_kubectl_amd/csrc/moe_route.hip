// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Mixture-of-experts routing with expert groups and a choice correction, and the experts of a few rows
// (models/kafilorn.py).
//
//   moe_route:  z = W_router h in fp32 (weights [E, W] fp32, one wave per logit); s = softmax(z) over all
//               experts, or (sigmoid) s = sigmoid(z) per expert; choice = s + correction (optional).  The experts form `groups` equal groups of
//               neighbours; a group's score is its largest choice; only experts of the `keep` best groups
//               can be chosen.  The `top` largest choices are taken (ties: the lower index); the weights
//               are their s (without the correction) over their sum (+ 1e-20), or (renorm 0) their s as they
//               are.  One workgroup per token.
//   moe_gate_up / moe_down:  for step sizes of a few rows (decode), the chosen experts as matrix-vector
//               products straight from the stacked expert weights, no routing lists and no host read, so a
//               decode step can be captured: act[t, k] = silu(gate_e h) * (up_e h) with e = ids[t, k], then
//               out[t] = sum_k w[t, k] down_e act[t, k] in fp32.  Any dtype; the fp32 engine's path.
//               in_scale: the weight multiplies the expert's INPUT instead of its output; as the two projections
//               are linear it is applied to their fp32 results, act = silu(w gate_e h) * (w up_e h), and the
//               outputs are summed as they are.
//   moe_grouped:  the same step in bf16 on the matrix cores, rows grouped by expert (below).
#include "rows_f32.h"

namespace {
using namespace rows;

constexpr int MAX_E = 1024;
constexpr int MAX_TOP = 32;

template <typename AT>
__global__ __launch_bounds__(NT) void moe_route_kernel(int* __restrict__ ids, float* __restrict__ wts,
                                                       const AT* __restrict__ h, const float* __restrict__ wr,
                                                       const float* __restrict__ correction, int width, int E, int top,
                                                       int groups, int keep, int sigmoid, int renorm) {
  __shared__ float z[MAX_E];      // logits, then scores
  __shared__ float ch[MAX_E];     // choice scores (minus infinity once taken or outside the kept groups)
  __shared__ float gs[MAX_E];     // group scores
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const AT* hr = h + (size_t)t * width;
  for (int e = wave; e < E; e += NW) {
    const float* we = wr + (size_t)e * width;
    float s = 0.f;
    if ((width & 7) == 0) {   // eight entries per lane and trip, 16-byte loads, four trips in flight
#pragma unroll 4
      for (int i = 8 * lane; i < width; i += 512) {
        const f32x4 wa = *reinterpret_cast<const f32x4*>(we + i), wb = *reinterpret_cast<const f32x4*>(we + i + 4);
        float x[8];
        if constexpr (sizeof(AT) == 2) {
          const uint4 hv = *reinterpret_cast<const uint4*>(hr + i);
          x[0] = lo_f(hv.x); x[1] = hi_f(hv.x); x[2] = lo_f(hv.y); x[3] = hi_f(hv.y);
          x[4] = lo_f(hv.z); x[5] = hi_f(hv.z); x[6] = lo_f(hv.w); x[7] = hi_f(hv.w);
        } else {
          const f32x4 ha = *reinterpret_cast<const f32x4*>(hr + i), hb = *reinterpret_cast<const f32x4*>(hr + i + 4);
          x[0] = ha[0]; x[1] = ha[1]; x[2] = ha[2]; x[3] = ha[3];
          x[4] = hb[0]; x[5] = hb[1]; x[6] = hb[2]; x[7] = hb[3];
        }
        s += x[0] * wa[0] + x[1] * wa[1] + x[2] * wa[2] + x[3] * wa[3] + x[4] * wb[0] + x[5] * wb[1] + x[6] * wb[2] + x[7] * wb[3];
      }
    } else {
      for (int i = lane; i < width; i += 64) s += ldf(hr + i) * we[i];
    }
    s = wave_sum(s);
    if (lane == 0) z[e] = s;
  }
  __syncthreads();
  if (wave != 0) return;
  float mx = -INFINITY, sum = 1.f;
  if (!sigmoid) {
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    sum = 0.f;
    for (int e = lane; e < E; e += 64) sum += expf(z[e] - mx);
    sum = wave_sum(sum);
  }
  for (int e = lane; e < E; e += 64) {
    const float s = sigmoid ? 1.0f / (1.0f + expf(-z[e])) : expf(z[e] - mx) / sum;
    z[e] = s;
    ch[e] = s + (correction != nullptr ? correction[e] : 0.f);
  }
  __builtin_amdgcn_wave_barrier();
  const int per = E / groups;
  if (groups > 1) {
    for (int g = lane; g < groups; g += 64) {
      float b = -INFINITY;
      for (int e = g * per; e < (g + 1) * per; ++e) b = fmaxf(b, ch[e]);
      gs[g] = b;
    }
    __builtin_amdgcn_wave_barrier();
    // a group is kept when fewer than `keep` groups come before it (larger score, or equal and lower index)
    for (int g = lane; g < groups; g += 64) {
      int before = 0;
      for (int o = 0; o < groups; ++o) before += (gs[o] > gs[g] || (gs[o] == gs[g] && o < g)) ? 1 : 0;
      if (before >= keep)
        for (int e = g * per; e < (g + 1) * per; ++e) ch[e] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
  }
  float wsum = 0.f, mine = 0.f;
  int mid = 0;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64)
      if (ch[e] > bv) { bv = ch[e]; bi = e; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi >= E) bi = 0;   // fewer finite choices than `top`: cannot happen for a valid router
    const float s = z[bi];
    wsum += s;
    if (lane == k % 64) { mine = s; mid = bi; }   // top <= MAX_TOP <= 64: lane k keeps the k-th choice
    if (lane == 0) ch[bi] = -INFINITY;
    __builtin_amdgcn_wave_barrier();
  }
  if (lane < top) {
    ids[(size_t)t * top + lane] = mid;
    wts[(size_t)t * top + lane] = renorm ? mine / (wsum + 1e-20f) : mine;
  }
}

// act[row, f] for row = t * top + k: one workgroup per (row, 4 * FPW outputs), h staged in LDS as fp32
constexpr int FPW = 4;   // outputs per wave
template <typename AT>
__global__ __launch_bounds__(NT) void moe_gate_up_kernel(AT* __restrict__ act, const AT* __restrict__ h,
                                                         const AT* __restrict__ w_gu, const int* __restrict__ ids,
                                                         const float* __restrict__ in_w, int width, int ff, int top) {
  extern __shared__ float hs[];   // [width]
  const int row = blockIdx.x, t = row / top;
  const int e = ids[row];
  const float isc = in_w != nullptr ? in_w[row] : 1.f;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < width; i += NT) hs[i] = ldf(h + (size_t)t * width + i);
  __syncthreads();
  const AT* wg = w_gu + (size_t)e * 2 * ff * width;
  for (int u = 0; u < FPW; ++u) {
    const int f = (blockIdx.y * NW + wave) * FPW + u;
    if (f >= ff) break;
    const AT* g = wg + (size_t)f * width;
    const AT* up = wg + (size_t)(ff + f) * width;
    float sg = 0.f, su = 0.f;
    for (int i = lane; i < width; i += 64) {
      sg += hs[i] * ldf(g + i);
      su += hs[i] * ldf(up + i);
    }
    sg = wave_sum(sg) * isc;
    su = wave_sum(su) * isc;
    if (lane == 0) stf(act + (size_t)row * ff + f, sg / (1.f + expf(-sg)) * su);
  }
}

// out[t, c] = sum_k w[t, k] * (down_e[c, :] . act[t * top + k, :]): one workgroup per (t, 4 * FPW columns)
template <typename AT>
__global__ __launch_bounds__(NT) void moe_down_kernel(float* __restrict__ out, const AT* __restrict__ act,
                                                      const AT* __restrict__ w_down, const int* __restrict__ ids,
                                                      const float* __restrict__ wts, int width, int ff, int top) {
  // wts null: the rows are summed as they are
  extern __shared__ float as[];   // [top][ff]
  __shared__ int se[MAX_TOP];
  __shared__ float sw[MAX_TOP];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < top * ff; i += NT) as[i] = ldf(act + (size_t)t * top * ff + i);
  if (threadIdx.x < top) {
    se[threadIdx.x] = ids[(size_t)t * top + threadIdx.x];
    sw[threadIdx.x] = wts != nullptr ? wts[(size_t)t * top + threadIdx.x] : 1.f;
  }
  __syncthreads();
  for (int u = 0; u < FPW; ++u) {
    const int c = (blockIdx.y * NW + wave) * FPW + u;
    if (c >= width) break;
    float s = 0.f;
    for (int k = 0; k < top; ++k) {
      const AT* d = w_down + ((size_t)se[k] * width + c) * ff;
      float p = 0.f;
      for (int i = lane; i < ff; i += 64) p += as[k * ff + i] * ldf(d + i);
      s += sw[k] * p;
    }
    s = wave_sum(s);
    if (lane == 0) out[(size_t)t * width + c] = s;
  }
}


// ---- bf16, matrix cores: the experts of a decode-sized step, grouped by expert so that every expert's weights
// are read once.  A workgroup takes (expert e, 64 output features): it lists the (token, choice) rows routed to e
// and runs them, 16 at a time, as the M rows of MFMA 16x16x32 products against the expert's weight rows (B
// fragments are 16-byte loads straight from the stacked weights, A fragments 16-byte loads of the gathered rows).
//   MODE 0: act[row] = silu(s gate_e x) * (s up_e x), x = h[row / top]     (bf16 out, K = width, N = ff;
//           s = in_w[row], or 1 when in_w is null)
//   MODE 1: yk[row]  = down_e act[row]                                      (fp32 out, K = ff,    N = width)
// and `moe_combine` sums a token's rows in the order of its choices with the router weights.  No host read and no
// data-dependent launch shape: a decode step with experts can be captured into a graph.
constexpr int GROUP_MAX_ROWS = 1024;

template <int MODE>
__global__ __launch_bounds__(NT) void moe_group_kernel(void* __restrict__ out, const bf16_t* __restrict__ x,
                                                       const bf16_t* __restrict__ w, const int* __restrict__ ids,
                                                       const float* __restrict__ in_w, int rows_, int K, int N, int top) {
  __shared__ int list[GROUP_MAX_ROWS];
  __shared__ int cnt;
  const int e = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  if (tid == 0) cnt = 0;
  __syncthreads();
  for (int r = tid; r < rows_; r += NT)
    if (ids[r] == e) list[atomicAdd(&cnt, 1)] = r;
  __syncthreads();
  const int n = cnt;
  if (n == 0) return;
  const int n0 = blockIdx.y * 64 + wave * 16;
  if (n0 >= N) return;
  const int nc = min(n0 + col, N - 1);
  const bf16_t* wg = w + ((size_t)e * (MODE == 0 ? 2 * N : N) + nc) * K + 8 * grp;
  const bf16_t* wu = wg + (size_t)N * K;   // MODE 0: the up rows follow the gate rows
  for (int mt = 0; mt * 16 < n; ++mt) {
    const int ridx = list[min(mt * 16 + col, n - 1)];
    const bf16_t* xr = x + (size_t)(MODE == 0 ? ridx / top : ridx) * K + 8 * grp;
    f32x4 ag = {0.f, 0.f, 0.f, 0.f}, au = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
    for (int k0 = 0; k0 < K; k0 += 32) {
      const bf16x8 a = as_bf16x8(*reinterpret_cast<const uint4*>(xr + k0));
      ag = mfma16x16x32(a, as_bf16x8(*reinterpret_cast<const uint4*>(wg + k0)), ag);
      if constexpr (MODE == 0) au = mfma16x16x32(a, as_bf16x8(*reinterpret_cast<const uint4*>(wu + k0)), au);
    }
    if (n0 + col < N) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = mt * 16 + 4 * grp + r;
        if (row < n) {
          const size_t at = (size_t)list[row] * N + n0 + col;
          if constexpr (MODE == 0) {
            const float isc = in_w != nullptr ? in_w[list[row]] : 1.f;
            const float gg = ag[r] * isc;
            reinterpret_cast<bf16_t*>(out)[at] = f2bf(gg / (1.f + expf(-gg)) * (au[r] * isc));
          } else {
            reinterpret_cast<float*>(out)[at] = ag[r];
          }
        }
      }
    }
  }
}

__global__ __launch_bounds__(NT) void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ yk,
                                                         const float* __restrict__ wts, int width, int top) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += NT) {
    float s = 0.f;
    for (int k = 0; k < top; ++k) s += (wts != nullptr ? wts[(size_t)t * top + k] : 1.f) * yk[((size_t)t * top + k) * width + c];
    out[(size_t)t * width + c] = s;
  }
}

}  // namespace

extern "C" int ka_moe_route(int* ids, float* wts, const void* h, const float* wr, const float* correction, int T,
                            int width, int E, int top, int groups, int keep, int sigmoid, int renorm, int f32,
                            hipStream_t st) {
  if (T <= 0) return 0;
  if (E <= 0 || E > MAX_E || top <= 0 || top > MAX_TOP || top > E || groups <= 0 || E % groups || keep <= 0 || keep > groups)
    return (int)hipErrorInvalidValue;
  if (f32)
    moe_route_kernel<float><<<T, NT, 0, st>>>(ids, wts, (const float*)h, wr, correction, width, E, top, groups, keep, sigmoid,
                                              renorm);
  else
    moe_route_kernel<bf16_t><<<T, NT, 0, st>>>(ids, wts, (const bf16_t*)h, wr, correction, width, E, top, groups, keep,
                                               sigmoid, renorm);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_moe_rows(float* out, void* act, const void* h, const void* w_gu, const void* w_down, const int* ids,
                           const float* wts, int T, int width, int ff, int top, int in_scale, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (top <= 0 || top > MAX_TOP || (size_t)width * 4 > 60 * 1024 || (size_t)top * ff * 4 > 60 * 1024)
    return (int)hipErrorInvalidValue;
  const int per = NW * FPW;
  dim3 g1(T * top, (ff + per - 1) / per), g2(T, (width + per - 1) / per);
  const size_t l1 = (size_t)width * sizeof(float), l2 = (size_t)top * ff * sizeof(float);
  const float* w_in = in_scale ? wts : nullptr;
  const float* w_out = in_scale ? nullptr : wts;
  if (f32) {
    moe_gate_up_kernel<float><<<g1, NT, l1, st>>>((float*)act, (const float*)h, (const float*)w_gu, ids, w_in, width, ff, top);
    moe_down_kernel<float><<<g2, NT, l2, st>>>(out, (const float*)act, (const float*)w_down, ids, w_out, width, ff, top);
  } else {
    moe_gate_up_kernel<bf16_t><<<g1, NT, l1, st>>>((bf16_t*)act, (const bf16_t*)h, (const bf16_t*)w_gu, ids, w_in, width, ff,
                                                   top);
    moe_down_kernel<bf16_t><<<g2, NT, l2, st>>>(out, (const bf16_t*)act, (const bf16_t*)w_down, ids, w_out, width, ff, top);
  }
  KA_CHECK_LAUNCH();
}

// bf16 only; `act` [T * top, ff] bf16 and `yk` [T * top, width] fp32 are scratch
extern "C" int ka_moe_grouped(float* out, void* act, float* yk, const void* h, const void* w_gu, const void* w_down,
                              const int* ids, const float* wts, int T, int width, int ff, int top, int E, int in_scale,
                              hipStream_t st) {
  if (T <= 0) return 0;
  if (T * top > GROUP_MAX_ROWS || width % 32 || ff % 32 || top <= 0 || E <= 0) return (int)hipErrorInvalidValue;
  moe_group_kernel<0><<<dim3(E, (ff + 63) / 64), NT, 0, st>>>(act, (const bf16_t*)h, (const bf16_t*)w_gu, ids,
                                                              in_scale ? wts : nullptr, T * top, width, ff, top);
  moe_group_kernel<1><<<dim3(E, (width + 63) / 64), NT, 0, st>>>(yk, (const bf16_t*)act, (const bf16_t*)w_down, ids, nullptr,
                                                                 T * top, ff, width, top);
  moe_combine_kernel<<<T, NT, 0, st>>>(out, yk, in_scale ? nullptr : wts, width, top);
  KA_CHECK_LAUNCH();
}
