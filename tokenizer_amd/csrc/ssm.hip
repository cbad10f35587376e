// Selective scan: per channel c and state n, S[c, n] <- exp(d_c A[c, n]) S[c, n] + d_c x_c B_n and y_c = sum_n S[c, n] C_n
// + D_c x_c over a batch of portions, with the state of every request in its slot, then y * silu(z).  Step sizes,
// exponentials, the state and the read-out are float in every dtype.  A state row starts with [channels * n] (S).
//
// Sixteen lanes share a channel, each with PER of its n numbers of state in registers; a workgroup has sixteen channels
// and walks tokens in order, sixteen at a time through LDS (the next sixteen are asked for while these are worked on).
// Short portions are walked whole.  Long ones are cut into chunks of `chunk` tokens that run side by side: every chunk
// but an entry's last first runs from zeros and leaves its end state and the sum of its step sizes; a second kernel
// carries the states from chunk to chunk (start of k + 1 = exp(A * sum of k) * start of k + end of k); then every
// chunk runs again from its true start and writes its rows, the last one the slot's state.
#include "common.h"

#define SS_LANES 16                    // lanes that share a channel
#define SS_CH (256 / SS_LANES)         // channels a workgroup
#define SS_STAGE 16                    // tokens that lie in LDS at a time
#define SS_MAX_PER 16                  // numbers of state a lane (n up to 256)

__device__ __forceinline__ float ss_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// x summed over the sixteen lanes of a row (lanes 16 i .. 16 i + 15), in every lane of the row: four rotations within
// the row, no trip through LDS.
__device__ __forceinline__ float ss_row_sum16(float x) {
#define SS_ROR(n) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x120 | (n), 0xF, 0xF, false))
  x += SS_ROR(8);
  x += SS_ROR(4);
  x += SS_ROR(2);
  x += SS_ROR(1);
#undef SS_ROR
  return x;
}

enum { SS_WHOLE = 0, SS_LOCAL = 1, SS_FINAL = 2 };

// x: rows of `x_stride`, channel c at c; pre: float [n_tokens, channels], the step sizes before softplus; A: float
// [channels, n]; low: rows of `low_stride` with B at b_off and C at c_off (n each); D: float [channels]; z: rows of
// `z_stride`, channel c at z_off + c; out: [n_tokens, channels].
// MODE SS_WHOLE: grid (entries, channel blocks): an entry's rows from the slot's state (zeros at position 0) to the slot's state.
// MODE SS_LOCAL: grid (entries, channel blocks, chunks): chunk k of an entry, unless it is the last, from zeros; its end
//   state goes to chunk_state[slot of the chunk] and the sum of its step sizes to chunk_sum; nothing else is written.
// MODE SS_FINAL: the same grid: chunk k from chunk_state[slot of the chunk] (its true start, put there by the carry), rows
//   written; the last chunk leaves the slot's state.
// The slot of chunk k of entry e is cu_q[e] / chunk + e + k (entries' chunks never meet: there are fewer than
// n_tokens / chunk + entries of them).
template <typename T, int PER, int MODE>
__global__ void __launch_bounds__(256)
selective_scan_kernel(const T* __restrict__ x, int x_stride, const float* __restrict__ pre, const float* __restrict__ A,
                      const T* __restrict__ low, int low_stride, int b_off, int c_off, const float* __restrict__ D,
                      const T* __restrict__ z, int z_stride, int z_off, float* __restrict__ state, size_t state_stride,
                      const int* __restrict__ cu_q, const int* __restrict__ first_position,
                      const int* __restrict__ state_slots, T* __restrict__ out, int channels, int n, int chunk,
                      float* __restrict__ chunk_state, float* __restrict__ chunk_sum) {
  constexpr int NP = PER * SS_LANES;                         // a row of B or C in LDS, filled up with zeros
  __shared__ float s_dt[SS_STAGE][SS_CH], s_x[SS_STAGE][SS_CH], s_z[SS_STAGE][SS_CH];
  __shared__ float s_b[SS_STAGE][NP], s_c[SS_STAGE][NP];
  const int e = blockIdx.x;
  const int lo_all = cu_q[e], hi_all = cu_q[e + 1];
  if (hi_all <= lo_all) return;                              // an entry that only fills the batch up
  int lo = lo_all, hi = hi_all;
  size_t at = 0;                                             // the chunk's slot
  if (MODE != SS_WHOLE) {
    lo = lo_all + (int)blockIdx.z * chunk;
    if (lo >= hi_all) return;
    hi = min(hi_all, lo + chunk);
    if (MODE == SS_LOCAL && hi == hi_all) return;            // nobody asks for the last chunk's end state from zeros
    at = (size_t)(lo_all / chunk + e + (int)blockIdx.z);
  }
  const int part = threadIdx.x % SS_LANES, mine = threadIdx.x / SS_LANES;
  const int c0 = blockIdx.y * SS_CH;
  const bool live = c0 + mine < channels;
  const int c = live ? c0 + mine : channels - 1;             // (lanes past the last channel walk along and store nothing)
  float* mem = state + (size_t)state_slots[e] * state_stride + (size_t)c * n;
  // (Only an entry of one chunk starts from the slot's row in the chunked form: the same workgroup then reads and writes
  // it.  The first of several chunks takes its start where the carry put it, since the last one writes the row.)
  const bool from_slot = MODE == SS_WHOLE || (MODE == SS_FINAL && lo == lo_all && hi == hi_all);
  const bool zeros = first_position[e] == 0;
  float S[PER], a[PER];
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = part + r * SS_LANES;
    const bool held = j < n;
    S[r] = 0.f;
    if (held && from_slot && !zeros) S[r] = mem[j];
    if (held && MODE == SS_FINAL && !from_slot) S[r] = chunk_state[(at * channels + c) * n + j];
    a[r] = held ? A[(size_t)c * n + j] : 0.f;
  }
  const float skip = D[c];
  float sum = 0.f;

  // What this thread brings of a stage: one (token, channel) of the step sizes, inputs and gates, and every 256th
  // number of the stage's B and C rows.
  const int f_token = threadIdx.x / SS_CH, f_channel = c0 + threadIdx.x % SS_CH;
  constexpr int BC = (SS_STAGE * NP + 255) / 256;
  float r_pre, r_x, r_z, r_b[BC], r_c[BC];
  auto fetch = [&](int t0) {
    const int t = t0 + f_token;
    const bool there = t < hi && f_channel < channels;
    r_pre = there ? pre[(size_t)t * channels + f_channel] : 0.f;
    r_x = there ? ld(x + (size_t)t * x_stride + f_channel) : 0.f;
    r_z = (there && MODE != SS_LOCAL) ? ld(z + (size_t)t * z_stride + z_off + f_channel) : 0.f;
#pragma unroll
    for (int i = 0; i < BC; ++i) {
      const int flat = threadIdx.x + i * 256, tt = flat / NP, j = flat % NP;
      const bool ok = tt < SS_STAGE && t0 + tt < hi && j < n;
      const T* row = low + (size_t)(ok ? t0 + tt : lo) * low_stride;
      r_b[i] = ok ? ld(row + b_off + j) : 0.f;
      r_c[i] = ok ? ld(row + c_off + j) : 0.f;
    }
  };

  // Where finished rows wait for the threads that write them out: sixteen tokens by sixteen channels.
  __shared__ float s_out[SS_STAGE][SS_CH];
  auto write_out = [&](int t0) {                             // thread (token, channel) of the stage that lies in s_out
    const int t = t0 + f_token;
    if (t < hi && f_channel < channels) st(out + (size_t)t * channels + f_channel, s_out[f_token][threadIdx.x % SS_CH]);
  };

  fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += SS_STAGE) {
    __syncthreads();                                         // the stage before has been read, its rows lie in s_out
    if (MODE != SS_LOCAL && t0 > lo) write_out(t0 - SS_STAGE);
    // (A token past the portion's end gets a step size of zero and zeros all round: it leaves the state as it is.)
    s_dt[f_token][threadIdx.x % SS_CH] = t0 + f_token < hi ? ss_softplus(r_pre) : 0.f;
    s_x[f_token][threadIdx.x % SS_CH] = r_x;
    s_z[f_token][threadIdx.x % SS_CH] = r_z;
#pragma unroll
    for (int i = 0; i < BC; ++i) {
      const int flat = threadIdx.x + i * 256;
      if (flat < SS_STAGE * NP) { s_b[flat / NP][flat % NP] = r_b[i]; s_c[flat / NP][flat % NP] = r_c[i]; }
    }
    __syncthreads();
    if (t0 + SS_STAGE < hi) fetch(t0 + SS_STAGE);            // under way while this stage is worked on
    float ys[SS_STAGE];
#pragma unroll
    for (int tt = 0; tt < SS_STAGE; ++tt) {
      const float step = s_dt[tt][mine], xv = s_x[tt][mine];
      const float in = step * xv;
      float y = 0.f;
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        const int j = part + r * SS_LANES;
        S[r] = fmaf(__expf(step * a[r]), S[r], in * s_b[tt][j]);
        y = fmaf(S[r], s_c[tt][j], y);
      }
      ys[tt] = y;
      if (MODE == SS_LOCAL) sum += step;
    }
    if (MODE != SS_LOCAL) {
      // Sixteen lanes hold sixteen tokens' parts each; four exchanges (with the lane 1, 2, 4 and 8 away, halving what is
      // held each time) leave lane i with token i's whole sum, which it gates and puts down.
#define SS_XOR1(v) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false))
#define SS_XOR2(v) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false))
#define SS_XOR8(v) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, false))
      const bool b0 = part & 1, b1 = part & 2, b2 = part & 4, b3 = part & 8;
      float v8[8], v4[4], v2[2];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float keep = b0 ? ys[2 * i + 1] : ys[2 * i], send = b0 ? ys[2 * i] : ys[2 * i + 1];
        v8[i] = keep + SS_XOR1(send);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float keep = b1 ? v8[2 * i + 1] : v8[2 * i], send = b1 ? v8[2 * i] : v8[2 * i + 1];
        v4[i] = keep + SS_XOR2(send);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const float keep = b2 ? v4[2 * i + 1] : v4[2 * i], send = b2 ? v4[2 * i] : v4[2 * i + 1];
        v2[i] = keep + __shfl_xor(send, 4, WAVE);
      }
      const float keep = b3 ? v2[1] : v2[0], send = b3 ? v2[0] : v2[1];
      const float y = keep + SS_XOR8(send);
#undef SS_XOR1
#undef SS_XOR2
#undef SS_XOR8
      const float gate = s_z[part][mine];
      s_out[part][mine] = fmaf(skip, s_x[part][mine], y) * (gate / (1.0f + __expf(-gate)));
    }
  }
  if (MODE != SS_LOCAL) {
    __syncthreads();
    write_out(lo + (hi - lo - 1) / SS_STAGE * SS_STAGE);
  }
  if (!live) return;
  if (MODE == SS_LOCAL) {
#pragma unroll
    for (int r = 0; r < PER; ++r)
      if (part + r * SS_LANES < n) chunk_state[(at * channels + c) * n + part + r * SS_LANES] = S[r];
    if (part == 0) chunk_sum[at * channels + c] = sum;
  } else if (hi == hi_all) {
#pragma unroll
    for (int r = 0; r < PER; ++r)
      if (part + r * SS_LANES < n) mem[part + r * SS_LANES] = S[r];
  }
}

// The states carried from chunk to chunk: a thread an (entry, channel, state) walks the entry's chunks; where a chunk's
// end state from zeros lay it leaves the chunk's true start.
__global__ void __launch_bounds__(256)
selective_carry_kernel(const float* __restrict__ A, const float* __restrict__ state, size_t state_stride,
                       const int* __restrict__ cu_q, const int* __restrict__ first_position,
                       const int* __restrict__ state_slots, int channels, int n, int chunk, float* __restrict__ chunk_state,
                       const float* __restrict__ chunk_sum) {
  const int e = blockIdx.x;
  const int lo = cu_q[e], hi = cu_q[e + 1];
  const int chunks = (hi - lo + chunk - 1) / chunk;
  if (chunks <= 1) return;                                   // (the one chunk starts from the slot's state itself)
  const size_t first = (size_t)(lo / chunk + e);
  for (int i = blockIdx.y * 256 + threadIdx.x; i < channels * n; i += gridDim.y * 256) {
    const int c = i / n;
    const float rate = A[i];
    float start = first_position[e] == 0 ? 0.f : state[(size_t)state_slots[e] * state_stride + i];
    for (int k = 0; k < chunks; ++k) {
      float* cell = chunk_state + (first + k) * channels * n + i;
      const float end = k + 1 < chunks ? *cell : 0.f;
      *cell = start;
      if (k + 1 < chunks) start = fmaf(__expf(rate * chunk_sum[(first + k) * channels + c]), start, end);
    }
  }
}

// chunk > 0: the chunked form, with room for n_tokens / chunk + n_entries chunks in chunk_state (float, channels * n a
// chunk) and chunk_sum (float, channels a chunk), and up to max_chunks chunks an entry.
extern "C" int ta_selective_scan(const void* x, int x_stride, const void* pre, const void* A, const void* low, int low_stride,
                                 int b_off, int c_off, const void* D, const void* z, int z_stride, int z_off, void* state,
                                 long state_stride, const void* cu_q, const void* first_position, const void* state_slots,
                                 void* out, int n_entries, int channels, int n, int dtype, int chunk, int max_chunks,
                                 void* chunk_state, void* chunk_sum, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (channels <= 0 || n <= 0 || n > SS_LANES * SS_MAX_PER || state_stride < (long)channels * n) return -1;
  if (chunk > 0 && (chunk % SS_STAGE || max_chunks <= 0 || !chunk_state || !chunk_sum)) return -1;
  const int blocks = (channels + SS_CH - 1) / SS_CH;
  const int per = (n + SS_LANES - 1) / SS_LANES;
#define SCAN(TT, PP, MM, GRID)                                                                                           \
  selective_scan_kernel<TT, PP, MM><<<GRID, 256, 0, stream>>>((const TT*)x, x_stride, (const float*)pre, (const float*)A, \
      (const TT*)low, low_stride, b_off, c_off, (const float*)D, (const TT*)z, z_stride, z_off, (float*)state,           \
      (size_t)state_stride, (const int*)cu_q, (const int*)first_position, (const int*)state_slots, (TT*)out, channels, n, \
      chunk, (float*)chunk_state, (float*)chunk_sum)
#define SCAN_SIZES(TT, MM, GRID)                                                                                         \
  if (per <= 1) SCAN(TT, 1, MM, GRID); else if (per <= 2) SCAN(TT, 2, MM, GRID); else if (per <= 4) SCAN(TT, 4, MM, GRID); \
  else if (per <= 8) SCAN(TT, 8, MM, GRID); else SCAN(TT, 16, MM, GRID)
#define SCAN_TYPES(MM, GRID) if (dtype == DT_F32) { SCAN_SIZES(float, MM, GRID); } else { SCAN_SIZES(bf16_t, MM, GRID); }
  if (chunk <= 0) {
    SCAN_TYPES(SS_WHOLE, dim3(n_entries, blocks));
    return LAUNCH_STATUS();
  }
  const dim3 grid(n_entries, blocks, max_chunks);
  SCAN_TYPES(SS_LOCAL, grid);
  int status = LAUNCH_STATUS();
  if (status) return status;
  const int carry_blocks = min(64, (channels * n + 255) / 256);
  selective_carry_kernel<<<dim3(n_entries, carry_blocks), 256, 0, stream>>>(
      (const float*)A, (const float*)state, (size_t)state_stride, (const int*)cu_q, (const int*)first_position,
      (const int*)state_slots, channels, n, chunk, (float*)chunk_state, (const float*)chunk_sum);
  status = LAUNCH_STATUS();
  if (status) return status;
  SCAN_TYPES(SS_FINAL, grid);
#undef SCAN_TYPES
#undef SCAN_SIZES
#undef SCAN
  return LAUNCH_STATUS();
}
