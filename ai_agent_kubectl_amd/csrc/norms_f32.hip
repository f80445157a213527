// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// Row kernels of the models that carry their residual stream in fp32 (models/vivepel.py): embedding
// gather into the fp32 stream, RMS norm in groups, the post-norm + layer-scale + residual-add (+ the
// next sublayer's pre-norm) in one pass, and the PolyNorm activation.  The statistics, the norm
// weights and the residual are fp32 whatever the activation type AT (bf16_t or float) is: AT is what
// the GEMMs before and after these kernels read and write.
//
//   group RMS norm:  the row is cut into `groups` equal consecutive parts; part g is divided by
//                    sqrt(mean(part_g^2) + eps); the whole row is multiplied by w.
//   post_norm_residual:  r += ls * gnorm(y; w_post)  (ls null: 1);   out_next = gnorm(r; w_next)   (optional)
//   PolyNorm:        out = a N(z) + b N(z^2) + c N(z^3) + e,  N(u) = u / sqrt(mean(u^2) + eps) per row.
#include "common.h"

namespace {

constexpr int NT = 256;
constexpr int MAX_GROUPS = 64;

template <typename T>
KA_DEV float ldf(const T* p) {
  if constexpr (sizeof(T) == 4) return *p;
  else return bf2f(*p);
}
template <typename T>
KA_DEV void stf(T* p, float v) {
  if constexpr (sizeof(T) == 4) *p = v;
  else *p = f2bf(v);
}

// sum over the block of up to three values per thread; every thread gets the totals
template <int N>
KA_DEV void block_sum(float (&v)[N], float* red /* [N * NT / 64] */) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < N; ++k) v[k] = wave_sum(v[k]);
  __syncthreads();   // red may still be read from the previous call
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < N; ++k) red[k * (NT / 64) + wave] = v[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < N; ++k) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) s += red[k * (NT / 64) + w];
    v[k] = s;
  }
}

// inv[g] = 1 / sqrt(mean(row_g^2) + eps) of the row staged in LDS
KA_DEV void group_stats(const float* row, int width, int groups, float eps, float* inv, float* red) {
  const int gsz = width / groups;
  for (int g = 0; g < groups; ++g) {
    float s[1] = {0.f};
    for (int i = threadIdx.x; i < gsz; i += NT) {
      const float x = row[g * gsz + i];
      s[0] += x * x;
    }
    block_sum<1>(s, red);
    if (threadIdx.x == 0) inv[g] = 1.0f / sqrtf(s[0] / (float)gsz + eps);
  }
  __syncthreads();
}

template <typename AT>
__global__ __launch_bounds__(NT) void embed_f32_kernel(float* __restrict__ out, const AT* __restrict__ table,
                                                       const int* __restrict__ ids, int width, int vocab) {
  const int row = blockIdx.x;
  int id = ids[row];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const AT* src = table + (size_t)id * width;
  for (int i = threadIdx.x; i < width; i += NT) out[(size_t)row * width + i] = ldf(src + i);
}

template <typename XT, typename OT>
__global__ __launch_bounds__(NT) void group_rmsnorm_kernel(OT* __restrict__ out, const XT* __restrict__ x,
                                                           const float* __restrict__ w, int width, int groups,
                                                           float eps) {
  extern __shared__ float lds[];
  float* row = lds;                 // [width]
  float* inv = lds + width;         // [MAX_GROUPS]
  float* red = inv + MAX_GROUPS;    // [3 * NT / 64]
  const size_t base = (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += NT) row[i] = ldf(x + base + i);
  __syncthreads();
  group_stats(row, width, groups, eps, inv, red);
  const int gsz = width / groups;
  for (int i = threadIdx.x; i < width; i += NT) stf(out + base + i, row[i] * inv[i / gsz] * w[i]);
}

template <typename YT, typename AT>   // YT: the sublayer's result (fp32 for a sum of experts), AT: the next norm's output
__global__ __launch_bounds__(NT) void post_norm_residual_kernel(float* __restrict__ resid, const YT* __restrict__ y,
                                                                const float* __restrict__ w_post,
                                                                const float* __restrict__ ls,
                                                                const float* __restrict__ w_next,
                                                                AT* __restrict__ out_next, int width, int groups,
                                                                float eps) {
  extern __shared__ float lds[];
  float* row = lds;
  float* inv = lds + width;
  float* red = inv + MAX_GROUPS;
  const size_t base = (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += NT) row[i] = ldf(y + base + i);
  __syncthreads();
  group_stats(row, width, groups, eps, inv, red);
  const int gsz = width / groups;
  for (int i = threadIdx.x; i < width; i += NT) {
    const float n = row[i] * inv[i / gsz] * w_post[i];
    const float r = resid[base + i] + (ls != nullptr ? ls[i] * n : n);
    resid[base + i] = r;
    row[i] = r;   // each thread rewrites only the entries it read
  }
  if (w_next == nullptr) return;
  __syncthreads();
  group_stats(row, width, groups, eps, inv, red);
  for (int i = threadIdx.x; i < width; i += NT) stf(out_next + base + i, row[i] * inv[i / gsz] * w_next[i]);
}

template <typename AT>
__global__ __launch_bounds__(NT) void polynorm_kernel(AT* __restrict__ out, const AT* __restrict__ z,
                                                      const float* __restrict__ coef, int ff, float eps) {
  __shared__ float red[3 * NT / 64];
  const size_t base = (size_t)blockIdx.x * ff;
  float s[3] = {0.f, 0.f, 0.f};
  for (int i = threadIdx.x; i < ff; i += NT) {
    const float v = ldf(z + base + i);
    const float v2 = v * v;
    s[0] += v2;
    s[1] += v2 * v2;
    s[2] += v2 * v2 * v2;
  }
  block_sum<3>(s, red);
  const float n = (float)ff;
  const float r1 = coef[0] / sqrtf(s[0] / n + eps);
  const float r2 = coef[1] / sqrtf(s[1] / n + eps);
  const float r3 = coef[2] / sqrtf(s[2] / n + eps);
  const float e = coef[3];
  for (int i = threadIdx.x; i < ff; i += NT) {
    const float v = ldf(z + base + i);
    const float v2 = v * v;
    stf(out + base + i, r1 * v + r2 * v2 + r3 * (v2 * v) + e);
  }
}

size_t row_lds(int width) { return (size_t)(width + MAX_GROUPS + 3 * NT / 64) * sizeof(float); }

bool row_ok(int rows, int width, int groups) {
  return rows >= 0 && width > 0 && groups > 0 && groups <= MAX_GROUPS && width % groups == 0 && row_lds(width) <= 64 * 1024;
}

}  // namespace

// f32: 1 when the activation type is float, 0 for bf16
extern "C" int ka_embed_f32(float* out, const void* table, const int* ids, int rows, int width, int vocab, int f32,
                            hipStream_t st) {
  if (rows <= 0) return 0;
  if (f32) embed_f32_kernel<float><<<rows, NT, 0, st>>>(out, (const float*)table, ids, width, vocab);
  else embed_f32_kernel<bf16_t><<<rows, NT, 0, st>>>(out, (const bf16_t*)table, ids, width, vocab);
  KA_CHECK_LAUNCH();
}

// x_f32: the input rows are float (the residual stream) whatever the output type is
extern "C" int ka_group_rmsnorm(void* out, const void* x, const float* w, int rows, int width, int groups, float eps,
                                int x_f32, int out_f32, hipStream_t st) {
  if (rows <= 0) return 0;
  if (!row_ok(rows, width, groups)) return (int)hipErrorInvalidValue;
  const size_t lds = row_lds(width);
  if (x_f32 && out_f32)
    group_rmsnorm_kernel<float, float><<<rows, NT, lds, st>>>((float*)out, (const float*)x, w, width, groups, eps);
  else if (x_f32)
    group_rmsnorm_kernel<float, bf16_t><<<rows, NT, lds, st>>>((bf16_t*)out, (const float*)x, w, width, groups, eps);
  else if (out_f32)
    group_rmsnorm_kernel<bf16_t, float><<<rows, NT, lds, st>>>((float*)out, (const bf16_t*)x, w, width, groups, eps);
  else
    group_rmsnorm_kernel<bf16_t, bf16_t><<<rows, NT, lds, st>>>((bf16_t*)out, (const bf16_t*)x, w, width, groups, eps);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_post_norm_residual(float* resid, const void* y, const float* w_post, const float* ls,
                                     const float* w_next, void* out_next, int rows, int width, int groups, float eps,
                                     int y_f32, int out_f32, hipStream_t st) {
  if (rows <= 0) return 0;
  if (!row_ok(rows, width, groups)) return (int)hipErrorInvalidValue;
  const size_t lds = row_lds(width);
  if (y_f32 && out_f32)
    post_norm_residual_kernel<float, float><<<rows, NT, lds, st>>>(resid, (const float*)y, w_post, ls, w_next,
                                                                  (float*)out_next, width, groups, eps);
  else if (y_f32)
    post_norm_residual_kernel<float, bf16_t><<<rows, NT, lds, st>>>(resid, (const float*)y, w_post, ls, w_next,
                                                                   (bf16_t*)out_next, width, groups, eps);
  else if (out_f32)
    post_norm_residual_kernel<bf16_t, float><<<rows, NT, lds, st>>>(resid, (const bf16_t*)y, w_post, ls, w_next,
                                                                   (float*)out_next, width, groups, eps);
  else
    post_norm_residual_kernel<bf16_t, bf16_t><<<rows, NT, lds, st>>>(resid, (const bf16_t*)y, w_post, ls, w_next,
                                                                    (bf16_t*)out_next, width, groups, eps);
  KA_CHECK_LAUNCH();
}

extern "C" int ka_polynorm(void* out, const void* z, const float* coef, int rows, int ff, float eps, int f32,
                           hipStream_t st) {
  if (rows <= 0) return 0;
  if (ff <= 0) return (int)hipErrorInvalidValue;
  if (f32) polynorm_kernel<float><<<rows, NT, 0, st>>>((float*)out, (const float*)z, coef, ff, eps);
  else polynorm_kernel<bf16_t><<<rows, NT, 0, st>>>((bf16_t*)out, (const bf16_t*)z, coef, ff, eps);
  KA_CHECK_LAUNCH();
}
