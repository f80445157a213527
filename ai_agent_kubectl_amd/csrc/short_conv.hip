// KA_HIP_LIB: mixers
// KA_HIPCC_FLAGS: -Xclang -target-feature -Xclang -packed-fp32-ops
// A short causal convolution over time, per channel, on columns of a projection row:
//
//   y_t[c] = sum_j w[c][j] * u_(t - taps + 1 + j)[c]        j = 0 .. taps - 1, the last tap meets the current row
//
// Rows of a sequence arrive in steps (a prompt portion of any length, or one decoded row).  Inputs from before
// the step come from the sequence's state slot, state[slot] [taps - 1, C]: its last taps - 1 inputs, newest last.
// Inputs before position 0 are zero, decided by the row's position and not by the state's content, so a slot is
// reused without clearing.  `short_conv` is two launches: the convolution (one workgroup per row, reads the old
// state), then the state's advance by the step's rows (one thread per sequence and channel: it reads the taps - 1
// values it needs into registers before it writes any).  The arithmetic of a row does not depend on how the
// sequence was cut into steps: the taps are summed in the same order from the same values.
// AT (bf16_t or float) is the type of the rows, the state and the result; the taps are fp32 and stored tap-major,
// w [taps, C], so that neighbouring channels' taps are neighbours; sums are fp32.  Steps with many rows in bf16
// take eight channels per thread in 16-byte pieces (the same sums in the same order).
#include "rows_f32.h"

namespace {
using namespace rows;

constexpr int MAX_TAPS = 8;

struct ConvArgs {
  const int* q_starts;    // [num_seqs + 1] or null (row t is sequence t)
  const int* seq_slots;   // [num_seqs] state slot, < 0: skip
  const int* positions;   // [T]
  int num_seqs, T;
  int ps, off, C, taps, act;
};

template <typename AT>
__global__ __launch_bounds__(NT) void short_conv_kernel(AT* __restrict__ out, const AT* __restrict__ proj,
                                                        const float* __restrict__ w, const AT* __restrict__ state,
                                                        ConvArgs a) {
  const int t = blockIdx.x;
  if (a.q_starts != nullptr && t >= a.q_starts[a.num_seqs]) return;   // padding rows past the last sequence
  const int seq = seq_of(a.q_starts, a.num_seqs, t);
  if (seq >= a.num_seqs) return;
  const int slot = a.seq_slots[seq];
  if (slot < 0) return;
  const int r = t - (a.q_starts ? a.q_starts[seq] : t);   // row of the step within its sequence
  const int p = a.positions[t];
  const int taps = a.taps, C = a.C;
  const AT* st = state != nullptr ? state + (size_t)slot * (taps - 1) * C : nullptr;
  for (int c = blockIdx.y * NT + threadIdx.x; c < C; c += gridDim.y * NT) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int d = taps - 1 - j;          // how many rows back
      if (p - d < 0) continue;             // before the sequence's start
      const float u = r - d >= 0 ? ldf(proj + (size_t)(t - d) * a.ps + a.off + c) : ldf(st + (size_t)(taps - 1 + r - d) * C + c);
      acc += w[(size_t)j * C + c] * u;
    }
    stf(out + (size_t)t * C + c, a.act ? acc / (1.f + expf(-acc)) : acc);
  }
}

// bf16, eight channels per thread: C, ps and off multiples of 8
__global__ __launch_bounds__(NT) void short_conv_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ proj,
                                                            const float* __restrict__ w, const bf16_t* __restrict__ state,
                                                            ConvArgs a) {
  const int t = blockIdx.x;
  if (a.q_starts != nullptr && t >= a.q_starts[a.num_seqs]) return;
  const int seq = seq_of(a.q_starts, a.num_seqs, t);
  if (seq >= a.num_seqs) return;
  const int slot = a.seq_slots[seq];
  if (slot < 0) return;
  const int r = t - (a.q_starts ? a.q_starts[seq] : t);
  const int p = a.positions[t];
  const int taps = a.taps, C = a.C;
  const bf16_t* st = state != nullptr ? state + (size_t)slot * (taps - 1) * C : nullptr;
  for (int c = 8 * (blockIdx.y * NT + threadIdx.x); c < C; c += 8 * gridDim.y * NT) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < taps; ++j) {
      const int d = taps - 1 - j;
      if (p - d < 0) continue;
      const bf16_t* src = r - d >= 0 ? proj + (size_t)(t - d) * a.ps + a.off + c : st + (size_t)(taps - 1 + r - d) * C + c;
      const uint4 u = *reinterpret_cast<const uint4*>(src);
      const f32x4 wa = *reinterpret_cast<const f32x4*>(w + (size_t)j * C + c), wb = *reinterpret_cast<const f32x4*>(w + (size_t)j * C + c + 4);
      acc[0] += wa[0] * lo_f(u.x);
      acc[1] += wa[1] * hi_f(u.x);
      acc[2] += wa[2] * lo_f(u.y);
      acc[3] += wa[3] * hi_f(u.y);
      acc[4] += wb[0] * lo_f(u.z);
      acc[5] += wb[1] * hi_f(u.z);
      acc[6] += wb[2] * lo_f(u.w);
      acc[7] += wb[3] * hi_f(u.w);
    }
    if (a.act) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = acc[i] / (1.f + expf(-acc[i]));
    }
    uint4 o;
    o.x = pack2(acc[0], acc[1]);
    o.y = pack2(acc[2], acc[3]);
    o.z = pack2(acc[4], acc[5]);
    o.w = pack2(acc[6], acc[7]);
    *reinterpret_cast<uint4*>(out + (size_t)t * C + c) = o;
  }
}

template <typename AT>
__global__ __launch_bounds__(NT) void short_conv_state_kernel(const AT* __restrict__ proj, AT* __restrict__ state,
                                                              ConvArgs a) {
  const int seq = blockIdx.x;
  const int slot = a.seq_slots[seq];
  if (slot < 0) return;
  const int r0 = a.q_starts ? a.q_starts[seq] : seq, r1 = a.q_starts ? a.q_starts[seq + 1] : seq + 1;
  const int n = r1 - r0;
  if (n <= 0) return;
  const int c = blockIdx.y * NT + threadIdx.x;
  if (c >= a.C) return;
  const int p0 = a.positions[r0], keep = a.taps - 1;
  AT* st = state + (size_t)slot * keep * a.C;
  AT v[MAX_TAPS - 1];
#pragma unroll
  for (int j = 0; j < MAX_TAPS - 1; ++j) {
    if (j < keep) {
      const int o = n - keep + j;          // row of the step (negative: from before it) that becomes entry j
      if (p0 + o < 0) stf(&v[j], 0.f);
      else if (o >= 0) v[j] = proj[(size_t)(r0 + o) * a.ps + a.off + c];
      else v[j] = st[(size_t)(keep + o) * a.C + c];
    }
  }
#pragma unroll
  for (int j = 0; j < MAX_TAPS - 1; ++j)
    if (j < keep) st[(size_t)j * a.C + c] = v[j];
}

}  // namespace

extern "C" int ka_short_conv(void* out, const void* proj, int ps, int off, int C, const float* w, int taps, void* state,
                             const int* seq_slots, const int* q_starts, int num_seqs, const int* positions, int T, int act,
                             int f32, hipStream_t st) {
  if (T <= 0 || num_seqs <= 0) return 0;
  if (C <= 0 || taps < 1 || taps > MAX_TAPS || off < 0 || off + C > ps || (taps > 1 && state == nullptr))
    return (int)hipErrorInvalidValue;
  ConvArgs a{q_starts, seq_slots, positions, num_seqs, T, ps, off, C, taps, act};
  const dim3 sgrid(num_seqs, (C + NT - 1) / NT);
  // few rows (a decode step): one channel per thread, so a thread's few dependent loads are the kernel's length
  const dim3 cgrid(T, T >= 1024 ? 1 : (C + NT - 1) / NT);
  if (f32) {
    short_conv_kernel<float><<<cgrid, NT, 0, st>>>((float*)out, (const float*)proj, w, (const float*)state, a);
    if (taps > 1) short_conv_state_kernel<float><<<sgrid, NT, 0, st>>>((const float*)proj, (float*)state, a);
  } else {
    const bool vec = C % 8 == 0 && ps % 8 == 0 && off % 8 == 0 && ((uintptr_t)proj & 15) == 0 && ((uintptr_t)out & 15) == 0 &&
                     ((uintptr_t)state & 15) == 0 && ((uintptr_t)w & 15) == 0;
    if (vec && T >= 1024)
      short_conv_vec_kernel<<<dim3(T, 1), NT, 0, st>>>((bf16_t*)out, (const bf16_t*)proj, w, (const bf16_t*)state, a);
    else
      short_conv_kernel<bf16_t><<<cgrid, NT, 0, st>>>((bf16_t*)out, (const bf16_t*)proj, w, (const bf16_t*)state, a);
    if (taps > 1) short_conv_state_kernel<bf16_t><<<sgrid, NT, 0, st>>>((const bf16_t*)proj, (bf16_t*)state, a);
  }
  KA_CHECK_LAUNCH();
}
