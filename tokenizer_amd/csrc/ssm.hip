// Selective scan: per channel c and state n, S[c, n] <- exp(d_c A[c, n]) S[c, n] + d_c x_c B_n and y_c = sum_n S[c, n] C_n
// + D_c x_c over a batch of portions, with the state of every request in its slot, then y * silu(z).  Step sizes,
// exponentials, the state and the read-out are float in every dtype.  A state row starts with [channels * n] (S).
#include "common.h"

#define SS_LANES 8           // lanes that share a channel: each keeps PER of the channel's n numbers of state

__device__ __forceinline__ float ss_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// x summed over the eight lanes 8 i .. 8 i + 7, in every one of them.
__device__ __forceinline__ float ss_sum8(float x) {
  x += __shfl_xor(x, 1, WAVE);
  x += __shfl_xor(x, 2, WAVE);
  x += __shfl_xor(x, 4, WAVE);
  return x;
}

// What a token brings for a lane: the channel's step size (before softplus), input and gate, and the lane's B and C.
template <int PER>
struct SsToken {
  float pre, x, z, B[PER], C[PER];
};

// x: rows of `x_stride`, channel c at c; pre: float [n_tokens, channels], the step sizes before softplus; A: float
// [channels, n]; low: rows of `low_stride` with B at b_off and C at c_off (n each); D: float [channels]; z: rows of
// `z_stride`, channel c at z_off + c; out: [n_tokens, channels].  A workgroup an (entry, 32 channels); lane (channel, j)
// keeps the states j, j + 8, ... of its channel in registers and walks the entry's tokens in order; a token's operands
// are asked for while the token before is worked on.
template <typename T, int PER>
__global__ void __launch_bounds__(256)
selective_scan_kernel(const T* __restrict__ x, int x_stride, const float* __restrict__ pre, const float* __restrict__ A,
                      const T* __restrict__ low, int low_stride, int b_off, int c_off, const float* __restrict__ D,
                      const T* __restrict__ z, int z_stride, int z_off, float* __restrict__ state, size_t state_stride,
                      const int* __restrict__ cu_q, const int* __restrict__ first_position,
                      const int* __restrict__ state_slots, T* __restrict__ out, int channels, int n) {
  const int e = blockIdx.x;
  const int lo = cu_q[e], hi = cu_q[e + 1];
  if (hi <= lo) return;                                      // an entry that only fills the batch up
  const int part = threadIdx.x % SS_LANES;
  const int c_raw = blockIdx.y * (256 / SS_LANES) + threadIdx.x / SS_LANES;
  const bool live = c_raw < channels;
  const int c = live ? c_raw : channels - 1;                 // (lanes past the last channel walk along and store nothing)
  float* mem = state + (size_t)state_slots[e] * state_stride + (size_t)c * n;
  const bool zeros = first_position[e] == 0;
  float S[PER], a[PER];
  bool held[PER];
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = part + r * SS_LANES;
    held[r] = j < n;
    S[r] = (held[r] && !zeros) ? mem[j] : 0.f;
    a[r] = held[r] ? A[(size_t)c * n + j] : 0.f;
  }
  const float skip = D[c];

  auto bring = [&](int t, SsToken<PER>& tok) {
    tok.pre = pre[(size_t)t * channels + c];
    tok.x = ld(x + (size_t)t * x_stride + c);
    tok.z = ld(z + (size_t)t * z_stride + z_off + c);
    const T* row = low + (size_t)t * low_stride;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int j = held[r] ? part + r * SS_LANES : 0;
      const float b = ld(row + b_off + j), cc = ld(row + c_off + j);
      tok.B[r] = held[r] ? b : 0.f;
      tok.C[r] = held[r] ? cc : 0.f;
    }
  };

  SsToken<PER> now, next;
  bring(lo, now);
  for (int t = lo; t < hi; ++t) {
    if (t + 1 < hi) bring(t + 1, next);
    const float step = ss_softplus(now.pre);
    const float in = step * now.x;
    float y = 0.f;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      S[r] = fmaf(expf(step * a[r]), S[r], in * now.B[r]);
      y = fmaf(S[r], now.C[r], y);
    }
    y = ss_sum8(y);
    if (part == 0 && live) {
      const float gate = now.z / (1.0f + expf(-now.z));
      st(out + (size_t)t * channels + c, fmaf(skip, now.x, y) * gate);
    }
    now = next;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < PER; ++r)
      if (held[r]) mem[part + r * SS_LANES] = S[r];
  }
}

extern "C" int ta_selective_scan(const void* x, int x_stride, const void* pre, const void* A, const void* low, int low_stride,
                                 int b_off, int c_off, const void* D, const void* z, int z_stride, int z_off, void* state,
                                 long state_stride, const void* cu_q, const void* first_position, const void* state_slots,
                                 void* out, int n_entries, int channels, int n, int dtype, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (channels <= 0 || n <= 0 || n > SS_LANES * 32 || state_stride < (long)channels * n) return -1;
  dim3 grid(n_entries, (channels + 256 / SS_LANES - 1) / (256 / SS_LANES));
  const int per = (n + SS_LANES - 1) / SS_LANES;
#define SCAN(TT, PP)                                                                                                     \
  selective_scan_kernel<TT, PP><<<grid, 256, 0, stream>>>((const TT*)x, x_stride, (const float*)pre, (const float*)A,     \
      (const TT*)low, low_stride, b_off, c_off, (const float*)D, (const TT*)z, z_stride, z_off, (float*)state,           \
      (size_t)state_stride, (const int*)cu_q, (const int*)first_position, (const int*)state_slots, (TT*)out, channels, n)
#define SCAN_SIZES(TT)                                                                                                   \
  if (per <= 1) SCAN(TT, 1); else if (per <= 2) SCAN(TT, 2); else if (per <= 3) SCAN(TT, 3); else if (per <= 4) SCAN(TT, 4); \
  else if (per <= 8) SCAN(TT, 8); else if (per <= 16) SCAN(TT, 16); else SCAN(TT, 32)
  if (dtype == DT_F32) { SCAN_SIZES(float); } else { SCAN_SIZES(bf16_t); }
#undef SCAN_SIZES
#undef SCAN
  return LAUNCH_STATUS();
}
