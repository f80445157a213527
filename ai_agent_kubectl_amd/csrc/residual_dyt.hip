// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Row kernels around an fp32 residual whose norm is Dynamic Tanh (models/suvapel.py).  One workgroup per row;
// the residual, the norm's slope / weight / bias and all arithmetic are fp32, AT (bf16_t or float) is the type
// the GEMMs before and after read and write.
//
//   dyt_norm:         h = tanh(alpha * x) * w + b                    no mean, no variance, alpha one learned number
//   residual_mix:     x += c0 y0 + c1 y1 + c2 y2                     the sublayers that read the same normed row;
//                     optionally x rounded to AT (the next GEMM's input) and / or dyt_norm(x) in the same pass
//   rms_residual:     x += mult * y / sqrt(mean(y^2) + eps) * w      optionally dyt_norm(x) in the same pass
//   gelu_gate_embed:  out = gelu_tanh(z) * table[id, col0 ...]       a gate on a slice of a second embedding row
//   silu_mul_bias:    out = silu(g + bg) * (u + bu)                  g | u columns of a wider projection row
#include "rows_f32.h"

namespace {
using namespace rows;

// elementwise row kernels: one workgroup per row when there are many rows, one entry per thread when there are few
// (a decode step), where a thread's chain of dependent loads is the kernel's length
inline dim3 row_grid(int rows_, int width) { return dim3(rows_, rows_ >= 1024 ? 1 : (width + NT - 1) / NT); }

KA_DEV float dyt(float x, float alpha, float w, float b) { return tanhf(alpha * x) * w + b; }

template <typename OT>
__global__ __launch_bounds__(NT) void dyt_norm_kernel(OT* __restrict__ out, const float* __restrict__ x,
                                                      const float* __restrict__ alpha, const float* __restrict__ w,
                                                      const float* __restrict__ b, int width) {
  const size_t base = (size_t)blockIdx.x * width;
  const float al = alpha[0];
  for (int i = blockIdx.y * NT + threadIdx.x; i < width; i += gridDim.y * NT) stf(out + base + i, dyt(x[base + i], al, w[i], b[i]));
}

template <typename YT, typename OT>
__global__ __launch_bounds__(NT) void residual_mix_kernel(float* __restrict__ x, const YT* __restrict__ y0,
                                                          const YT* __restrict__ y1, const YT* __restrict__ y2, float c0,
                                                          float c1, float c2, OT* __restrict__ copy, OT* __restrict__ h,
                                                          const float* __restrict__ alpha, const float* __restrict__ w,
                                                          const float* __restrict__ b, int width) {
  const size_t base = (size_t)blockIdx.x * width;
  const float al = h != nullptr ? alpha[0] : 0.f;
  for (int i = blockIdx.y * NT + threadIdx.x; i < width; i += gridDim.y * NT) {
    float s = c0 * ldf(y0 + base + i);
    if (y1 != nullptr) s += c1 * ldf(y1 + base + i);
    if (y2 != nullptr) s += c2 * ldf(y2 + base + i);
    const float v = x[base + i] + s;
    x[base + i] = v;
    if (copy != nullptr) stf(copy + base + i, v);
    if (h != nullptr) stf(h + base + i, dyt(v, al, w[i], b[i]));
  }
}

template <typename YT, typename OT>
__global__ __launch_bounds__(NT) void rms_residual_kernel(float* __restrict__ x, const YT* __restrict__ y,
                                                          const float* __restrict__ wn, float mult, float eps,
                                                          OT* __restrict__ h, const float* __restrict__ alpha,
                                                          const float* __restrict__ w, const float* __restrict__ b,
                                                          int width) {
  __shared__ float red[NW];
  const size_t base = (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    const float v = ldf(y + base + i);
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)width + eps);
  const float al = h != nullptr ? alpha[0] : 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    const float v = x[base + i] + mult * (ldf(y + base + i) * inv * wn[i]);
    x[base + i] = v;
    if (h != nullptr) stf(h + base + i, dyt(v, al, w[i], b[i]));
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void gelu_gate_embed_kernel(AT* __restrict__ out, const AT* __restrict__ z,
                                                             const AT* __restrict__ table, const int* __restrict__ ids,
                                                             int dim, int stride, int col0, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const AT* e = table + (size_t)id * stride + col0;
  for (int i = threadIdx.x; i < dim; i += NT) {
    const float v = ldf(z + (size_t)t * dim + i);
    const float g = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    stf(out + (size_t)t * dim + i, g * ldf(e + i));
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void silu_mul_bias_kernel(AT* __restrict__ out, const AT* __restrict__ proj, int ps,
                                                           int off, int ff, const float* __restrict__ bias) {
  const AT* g = proj + (size_t)blockIdx.x * ps + off;
  AT* o = out + (size_t)blockIdx.x * ff;
  for (int i = blockIdx.y * NT + threadIdx.x; i < ff; i += gridDim.y * NT) {
    const float a = ldf(g + i) + bias[i];
    stf(o + i, a / (1.f + expf(-a)) * (ldf(g + ff + i) + bias[ff + i]));
  }
}

}  // namespace

extern "C" int ka_dyt_norm(void* out, const float* x, const float* alpha, const float* w, const float* b, int rows_,
                           int width, int out_f32, hipStream_t st) {
  if (rows_ <= 0) return 0;
  if (width <= 0) return (int)hipErrorInvalidValue;
  if (out_f32) dyt_norm_kernel<float><<<row_grid(rows_, width), NT, 0, st>>>((float*)out, x, alpha, w, b, width);
  else dyt_norm_kernel<bf16_t><<<row_grid(rows_, width), NT, 0, st>>>((bf16_t*)out, x, alpha, w, b, width);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_residual_mix(float* x, const void* y0, const void* y1, const void* y2, float c0, float c1, float c2,
                               void* copy, void* h, const float* alpha, const float* w, const float* b, int rows_,
                               int width, int y_f32, int out_f32, hipStream_t st) {
  if (rows_ <= 0) return 0;
  if (width <= 0 || y0 == nullptr) return (int)hipErrorInvalidValue;
#define KA_RM(YT, OT)                                                                                                  \
  residual_mix_kernel<YT, OT><<<row_grid(rows_, width), NT, 0, st>>>(x, (const YT*)y0, (const YT*)y1, (const YT*)y2, c0, c1, c2, (OT*)copy, \
                                                    (OT*)h, alpha, w, b, width)
  if (y_f32 && out_f32) KA_RM(float, float);
  else if (y_f32) KA_RM(float, bf16_t);
  else if (out_f32) KA_RM(bf16_t, float);
  else KA_RM(bf16_t, bf16_t);
#undef KA_RM
  KA_CHECK_LAUNCH();
}

extern "C" int ka_rms_residual(float* x, const void* y, const float* wn, float mult, float eps, void* h,
                               const float* alpha, const float* w, const float* b, int rows_, int width, int y_f32,
                               int out_f32, hipStream_t st) {
  if (rows_ <= 0) return 0;
  if (width <= 0) return (int)hipErrorInvalidValue;
#define KA_RR(YT, OT) \
  rms_residual_kernel<YT, OT><<<rows_, NT, 0, st>>>(x, (const YT*)y, wn, mult, eps, (OT*)h, alpha, w, b, width)
  if (y_f32 && out_f32) KA_RR(float, float);
  else if (y_f32) KA_RR(float, bf16_t);
  else if (out_f32) KA_RR(bf16_t, float);
  else KA_RR(bf16_t, bf16_t);
#undef KA_RR
  KA_CHECK_LAUNCH();
}

extern "C" int ka_gelu_gate_embed(void* out, const void* z, const void* table, const int* ids, int rows_, int dim,
                                  int stride, int col0, int vocab, int f32, hipStream_t st) {
  if (rows_ <= 0) return 0;
  if (dim <= 0 || col0 < 0 || col0 + dim > stride || vocab <= 0) return (int)hipErrorInvalidValue;
  if (f32)
    gelu_gate_embed_kernel<float><<<rows_, NT, 0, st>>>((float*)out, (const float*)z, (const float*)table, ids, dim,
                                                        stride, col0, vocab);
  else
    gelu_gate_embed_kernel<bf16_t><<<rows_, NT, 0, st>>>((bf16_t*)out, (const bf16_t*)z, (const bf16_t*)table, ids, dim,
                                                         stride, col0, vocab);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_silu_mul_bias(void* out, const void* proj, int ps, int off, int ff, const float* bias, int rows_,
                                int f32, hipStream_t st) {
  if (rows_ <= 0) return 0;
  if (ff <= 0 || off < 0 || off + 2 * ff > ps) return (int)hipErrorInvalidValue;
  if (f32) silu_mul_bias_kernel<float><<<row_grid(rows_, ff), NT, 0, st>>>((float*)out, (const float*)proj, ps, off, ff, bias);
  else silu_mul_bias_kernel<bf16_t><<<row_grid(rows_, ff), NT, 0, st>>>((bf16_t*)out, (const bf16_t*)proj, ps, off, ff, bias);
  KA_CHECK_LAUNCH();
}
