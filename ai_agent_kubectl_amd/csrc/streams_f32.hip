// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Residual streams (hyper-connections) in fp32 and the row kernels around them (models/kafilorn.py).
// The residual is S copies x[t, s, :] of the row.  A sublayer reads one mixed row and writes all copies:
//
//   stream_norm:    u = sum_s w_in[s] x[t, s];   h = (u - mean u) / sqrt(var u + eps) * w     (LayerNorm, no bias)
//   stream_update:  x[t, r] <- sum_s mix[s, r] x[t, s] + out[r] * y[t]   for all r from the old copies, in one
//                   pass, and (optionally) the next sublayer's stream_norm of the new copies in the same pass.
//
// S = 1 with w_in = mix = out = 1 is the plain pre-norm residual.  Also here: the embedding gather into
// the S copies with a scale, relu(z)^2, silu(gate) * up (optionally of a row whose input was multiplied by a number
// s: silu(s gate) * (s up)), the clamped gated unit g sigmoid(alpha g) (u + 1) with g = min(gate, limit) and
// u = clamp(up, -limit, limit), and the per-head RMS division with an output
// gate that closes an mLSTM (o <- o / den; out = o / rms_head(o) * w * sigmoid(g)).
#include "rows_f32.h"

namespace {
using namespace rows;

constexpr int MAX_STREAMS = 16;

template <typename AT>
__global__ __launch_bounds__(NT) void embed_streams_kernel(float* __restrict__ out, const AT* __restrict__ table,
                                                           const int* __restrict__ ids, int width, int vocab,
                                                           float scale, int S) {
  const int row = blockIdx.x;
  int id = ids[row];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const AT* src = table + (size_t)id * width;
  float* dst = out + (size_t)row * S * width;
  for (int i = threadIdx.x; i < width; i += NT) {
    const float v = ldf(src + i) * scale;
    for (int s = 0; s < S; ++s) dst[(size_t)s * width + i] = v;
  }
}

// LayerNorm of the row staged in LDS (two passes: mean, then the mean of squared deviations)
template <typename OT>
KA_DEV void layer_norm_row(const float* row, int width, const float* __restrict__ w, float eps, OT* __restrict__ out,
                           float* red) {
  float s = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) s += row[i];
  const float mean = block_sum(s, red) / (float)width;
  float q = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    const float d = row[i] - mean;
    q += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum(q, red) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += NT) stf(out + i, (row[i] - mean) * inv * w[i]);
}

template <typename OT>
__global__ __launch_bounds__(NT) void stream_norm_kernel(OT* __restrict__ out, const float* __restrict__ x,
                                                         const float* __restrict__ w_in, const float* __restrict__ w,
                                                         int width, int S, float eps) {
  extern __shared__ float lds[];
  float* row = lds;            // [width]
  float* red = lds + width;    // [NW]
  const float* xr = x + (size_t)blockIdx.x * S * width;
#pragma unroll 4
  for (int i = threadIdx.x; i < width; i += NT) {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u += w_in[s] * xr[(size_t)s * width + i];
    row[i] = u;
  }
  __syncthreads();
  layer_norm_row(row, width, w, eps, out + (size_t)blockIdx.x * width, red);
}

template <typename YT, typename OT>
__global__ __launch_bounds__(NT) void stream_update_kernel(float* __restrict__ x, const YT* __restrict__ y,
                                                           const float* __restrict__ mix, const float* __restrict__ outw,
                                                           const float* __restrict__ next_in,
                                                           const float* __restrict__ next_w, OT* __restrict__ out_next,
                                                           int width, int S, float eps) {
  extern __shared__ float lds[];
  float* row = lds;
  float* red = lds + width;
  __shared__ float smix[MAX_STREAMS * MAX_STREAMS], sout[MAX_STREAMS], snin[MAX_STREAMS];
  if (threadIdx.x < S * S) smix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    sout[threadIdx.x] = outw[threadIdx.x];
    snin[threadIdx.x] = next_in != nullptr ? next_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  float* xr = x + (size_t)blockIdx.x * S * width;
  const YT* yr = y + (size_t)blockIdx.x * width;
#pragma unroll 4
  for (int i = threadIdx.x; i < width; i += NT) {
    float old[MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s) old[s] = s < S ? xr[(size_t)s * width + i] : 0.f;
    const float yv = ldf(yr + i);
    float u = 0.f;
#pragma unroll
    for (int r = 0; r < MAX_STREAMS; ++r) {
      if (r < S) {
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s)
          if (s < S) v += smix[s * S + r] * old[s];
        v += sout[r] * yv;
        xr[(size_t)r * width + i] = v;
        u += snin[r] * v;
      }
    }
    row[i] = u;
  }
  if (next_w == nullptr) return;
  __syncthreads();
  layer_norm_row(row, width, next_w, eps, out_next + (size_t)blockIdx.x * width, red);
}

template <typename AT>
__global__ __launch_bounds__(NT) void relu_sq_kernel(AT* __restrict__ out, const AT* __restrict__ z, size_t n) {
  for (size_t i = (size_t)blockIdx.x * NT + threadIdx.x; i < n; i += (size_t)gridDim.x * NT) {
    const float v = fmaxf(ldf(z + i), 0.f);
    stf(out + i, v * v);
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void silu_mul_rows_kernel(AT* __restrict__ out, const AT* __restrict__ gu,
                                                           const float* __restrict__ row_scale, int ff) {
  const AT* g = gu + (size_t)blockIdx.x * 2 * ff;
  AT* o = out + (size_t)blockIdx.x * ff;
  const float sc = row_scale != nullptr ? row_scale[blockIdx.x] : 1.f;
  for (int i = threadIdx.x; i < ff; i += NT) {
    const float a = ldf(g + i) * sc;
    stf(o + i, a / (1.f + expf(-a)) * (ldf(g + ff + i) * sc));
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void glu_clamp_kernel(AT* __restrict__ out, const AT* __restrict__ gu, int ff, float limit,
                                                       float alpha) {
  const AT* g = gu + (size_t)blockIdx.x * 2 * ff;
  AT* o = out + (size_t)blockIdx.x * ff;
  for (int i = threadIdx.x + blockIdx.y * NT; i < ff; i += NT * gridDim.y) {
    const float a = fminf(ldf(g + i), limit);
    const float u = fminf(fmaxf(ldf(g + ff + i), -limit), limit);
    stf(o + i, a / (1.f + expf(-alpha * a)) * (u + 1.f));
  }
}

// one wave per head: o [T, H * Dv] fp32 -> out in AT; the gate columns sit in `proj` rows of stride ps at g_off
// (sigmoid of them, or silu of them)
// den [T, H] (optional): the head's entries are first divided by den[t, h]
template <typename AT>
__global__ __launch_bounds__(NT) void headnorm_gate_kernel(AT* __restrict__ out, const float* __restrict__ o,
                                                           const float* __restrict__ den, const AT* __restrict__ proj,
                                                           int ps, int g_off, const float* __restrict__ w, int H, int Dv,
                                                           float eps, int silu) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int h = wave; h < H; h += NW) {
    const float* oh = o + ((size_t)t * H + h) * Dv;
    const float rd = den != nullptr ? 1.0f / den[(size_t)t * H + h] : 1.0f;
    float ss = 0.f;
    for (int i = lane; i < Dv; i += 64) {
      const float v = oh[i] * rd;
      ss += v * v;
    }
    const float inv = rd / sqrtf(wave_sum(ss) / (float)Dv + eps);
    for (int i = lane; i < Dv; i += 64) {
      const float g = ldf(proj + (size_t)t * ps + g_off + h * Dv + i);
      stf(out + ((size_t)t * H + h) * Dv + i, oh[i] * inv * w[h * Dv + i] * (silu ? g : 1.f) / (1.f + expf(-g)));
    }
  }
}

}  // namespace

extern "C" int ka_embed_streams(float* out, const void* table, const int* ids, int T, int width, int vocab, float scale,
                                int S, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (S <= 0 || width <= 0) return (int)hipErrorInvalidValue;
  if (f32) embed_streams_kernel<float><<<T, NT, 0, st>>>(out, (const float*)table, ids, width, vocab, scale, S);
  else embed_streams_kernel<bf16_t><<<T, NT, 0, st>>>(out, (const bf16_t*)table, ids, width, vocab, scale, S);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_stream_norm(void* out, const float* x, const float* w_in, const float* w, int rows_, int width, int S,
                              float eps, int out_f32, hipStream_t st) {
  if (rows_ <= 0) return 0;
  const size_t lds = (size_t)(width + NW) * sizeof(float);
  if (S <= 0 || S > MAX_STREAMS || lds > 60 * 1024) return (int)hipErrorInvalidValue;
  if (out_f32) stream_norm_kernel<float><<<rows_, NT, lds, st>>>((float*)out, x, w_in, w, width, S, eps);
  else stream_norm_kernel<bf16_t><<<rows_, NT, lds, st>>>((bf16_t*)out, x, w_in, w, width, S, eps);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_stream_update(float* x, const void* y, const float* mix, const float* outw, const float* next_in,
                                const float* next_w, void* out_next, int rows_, int width, int S, float eps, int y_f32,
                                int out_f32, hipStream_t st) {
  if (rows_ <= 0) return 0;
  const size_t lds = (size_t)(width + NW) * sizeof(float);
  if (S <= 0 || S > MAX_STREAMS || lds > 60 * 1024) return (int)hipErrorInvalidValue;
#define KA_SU(YT, OT) \
  stream_update_kernel<YT, OT><<<rows_, NT, lds, st>>>(x, (const YT*)y, mix, outw, next_in, next_w, (OT*)out_next, width, S, eps)
  if (y_f32 && out_f32) KA_SU(float, float);
  else if (y_f32) KA_SU(float, bf16_t);
  else if (out_f32) KA_SU(bf16_t, float);
  else KA_SU(bf16_t, bf16_t);
#undef KA_SU
  KA_CHECK_LAUNCH();
}

extern "C" int ka_relu_sq(void* out, const void* z, long n, int f32, hipStream_t st) {
  if (n <= 0) return 0;
  const int grid = (int)((n + NT * 4 - 1) / (NT * 4) < 65535 * 8 ? (n + NT * 4 - 1) / (NT * 4) : 65535 * 8);
  if (f32) relu_sq_kernel<float><<<grid, NT, 0, st>>>((float*)out, (const float*)z, (size_t)n);
  else relu_sq_kernel<bf16_t><<<grid, NT, 0, st>>>((bf16_t*)out, (const bf16_t*)z, (size_t)n);
  KA_CHECK_LAUNCH();
}

// row_scale [rows] or null
extern "C" int ka_silu_mul_rows(void* out, const void* gu, const float* row_scale, int rows_, int ff, int f32,
                                hipStream_t st) {
  if (rows_ <= 0) return 0;
  if (f32) silu_mul_rows_kernel<float><<<rows_, NT, 0, st>>>((float*)out, (const float*)gu, row_scale, ff);
  else silu_mul_rows_kernel<bf16_t><<<rows_, NT, 0, st>>>((bf16_t*)out, (const bf16_t*)gu, row_scale, ff);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_glu_clamp(void* out, const void* gu, int rows_, int ff, float limit, float alpha, int f32, hipStream_t st) {
  if (rows_ <= 0) return 0;
  if (ff <= 0) return (int)hipErrorInvalidValue;
  // few rows (a decode step): a row's entries are spread over several workgroups
  const dim3 grid(rows_, rows_ < 1024 ? (ff + 4 * NT - 1) / (4 * NT) : 1);
  if (f32) glu_clamp_kernel<float><<<grid, NT, 0, st>>>((float*)out, (const float*)gu, ff, limit, alpha);
  else glu_clamp_kernel<bf16_t><<<grid, NT, 0, st>>>((bf16_t*)out, (const bf16_t*)gu, ff, limit, alpha);
  KA_CHECK_LAUNCH();
}

// silu: the gate is silu(g) = g * sigmoid(g) instead of sigmoid(g)
extern "C" int ka_headnorm_gate(void* out, const float* o, const float* den, const void* proj, int ps, int g_off,
                                const float* w, int T, int H, int Dv, float eps, int silu, int f32, hipStream_t st) {
  if (T <= 0) return 0;
  if (f32) headnorm_gate_kernel<float><<<T, NT, 0, st>>>((float*)out, o, den, (const float*)proj, ps, g_off, w, H, Dv, eps, silu);
  else headnorm_gate_kernel<bf16_t><<<T, NT, 0, st>>>((bf16_t*)out, o, den, (const bf16_t*)proj, ps, g_off, w, H, Dv, eps, silu);
  KA_CHECK_LAUNCH();
}
