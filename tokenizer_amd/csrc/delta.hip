// Gated delta rule with a decay per key channel, over a batch of portions, with the state of every request in its
// slot: the short causal convolutions in front of it (with silu) and the recurrence itself.  Unit vectors, gates,
// decays and the state are float in every dtype.  A state row is
// [heads * d * dv (S, per head [d, dv]) | (taps - 1) * channels (the convolutions' last inputs, oldest first) | ...].
#include "common.h"

#define DL_GROUP 16          // tokens whose q, k, decays (and v) are brought into LDS in one trip
#define DL_MAX_D 256
#define DL_MAX_TAPS 16

// x summed over the sixteen lanes of a row (lanes 16 i .. 16 i + 15), in every lane of the row: four rotations within the
// row, which cost no trip through LDS.
__device__ __forceinline__ float dl_row_sum16(float x) {
#define DL_ROR(n) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x120 | (n), 0xF, 0xF, false))
  x += DL_ROR(8);
  x += DL_ROR(4);
  x += DL_ROR(2);
  x += DL_ROR(1);
#undef DL_ROR
  return x;
}

__device__ __forceinline__ float dl_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// Up to three runs of columns of `rows` (run i: `width[i]` columns from `offset[i]` on) are the channels, side by side.
struct ConvRuns { int offset[3]; int width[3]; };

__device__ __forceinline__ int conv_column(const ConvRuns& runs, int c) {
  if (c < runs.width[0]) return runs.offset[0] + c;
  c -= runs.width[0];
  if (c < runs.width[1]) return runs.offset[1] + c;
  return runs.offset[2] + c - runs.width[1];
}

// out[t, c] = silu(bias[c] + sum_j taps[c, j] * x[t - (n_taps - 1) + j, c]) (bias float [channels], or null): inputs before the portion's first row come from the
// entry's state row (its last n_taps - 1 inputs, oldest first), and are zeros if the portion starts at position 0.
// A thread a (token, channel); blockIdx.x is the token.
template <typename T>
__global__ void __launch_bounds__(256)
short_conv_silu_kernel(const T* __restrict__ rows, int row_stride, ConvRuns runs, int channels, const float* __restrict__ taps,
                       int n_taps, const float* __restrict__ state, size_t state_stride, int state_offset,
                       const int* __restrict__ cu_q, const int* __restrict__ first_position,
                       const int* __restrict__ state_slots, const int* __restrict__ entry_of_token, T* __restrict__ out,
                       const float* __restrict__ bias) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int e = entry_of_token[t];
  if (e < 0) {                                               // a token that only fills the batch up
    st(out + (size_t)t * channels + c, 0.f);
    return;
  }
  const int lo = cu_q[e];
  const bool zeros = first_position[e] == 0;
  const float* tail = state + (size_t)state_slots[e] * state_stride + state_offset;
  const int column = conv_column(runs, c);
  float y = bias ? bias[c] : 0.f;
  for (int j = 0; j < n_taps; ++j) {
    const int src = t - (n_taps - 1) + j;
    float x;
    if (src >= lo) x = ld(rows + (size_t)src * row_stride + column);
    else x = zeros ? 0.f : tail[(size_t)(src - lo + n_taps - 1) * channels + c];
    y = fmaf(taps[(size_t)c * n_taps + j], x, y);
  }
  st(out + (size_t)t * channels + c, y / (1.0f + expf(-y)));
}

// The entry's last n_taps - 1 inputs become its state row's: a thread an (entry, channel) moves what stays of the old
// ones forward (reading ahead of what it writes) and puts the portion's last rows behind them.
template <typename T>
__global__ void __launch_bounds__(256)
short_conv_keep_kernel(const T* __restrict__ rows, int row_stride, ConvRuns runs, int channels, int n_taps,
                       float* __restrict__ state, size_t state_stride, int state_offset, const int* __restrict__ cu_q,
                       const int* __restrict__ first_position, const int* __restrict__ state_slots) {
  const int e = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int lo = cu_q[e], hi = cu_q[e + 1], n = hi - lo, keep = n_taps - 1;
  if (n <= 0) return;
  const bool zeros = first_position[e] == 0;
  float* tail = state + (size_t)state_slots[e] * state_stride + state_offset;
  const int column = conv_column(runs, c);
  for (int i = 0; i < keep; ++i) {
    const int at = i + n;                          // the place in [old inputs | the portion's rows]
    float x;
    if (at < keep) x = zeros ? 0.f : tail[(size_t)at * channels + c];
    else x = ld(rows + (size_t)(lo + at - keep) * row_stride + column);
    tail[(size_t)i * channels + c] = x;
  }
}

// What the recurrence needs of a token that does not depend on the state, for every token side by side: q and k as unit
// vectors per query/key head (q times d^(-1/2)) and their product, the decays g = exp(neg_rate * softplus(z)) in place
// of their pre-activations z, and beta = sigmoid(.).  A workgroup a token; a wave a query/key head at a time.
// prep: float rows of 2 groups d + heads + groups: [q | k | beta | q . k].
template <typename T>
__global__ void __launch_bounds__(4 * WAVE)
delta_prepare_kernel(const T* __restrict__ fresh, int fresh_stride, float* __restrict__ z, const float* __restrict__ neg_rate,
                     const T* __restrict__ beta_rows, int beta_stride, int beta_offset, float* __restrict__ prep, int heads,
                     int groups, int d, float unit_eps) {
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int width = 2 * groups * d + heads + groups;
  const T* x = fresh + (size_t)t * fresh_stride;
  float* out = prep + (size_t)t * width;
  const float q_scale = 1.0f / sqrtf((float)d);
  for (int g = wave; g < groups; g += 4) {
    float sq = 0.f, sk = 0.f, qk = 0.f;
    for (int j = lane; j < d; j += WAVE) {
      const float qv = ld(x + (size_t)g * d + j), kv = ld(x + (size_t)(groups + g) * d + j);
      sq = fmaf(qv, qv, sq);
      sk = fmaf(kv, kv, sk);
      qk = fmaf(qv, kv, qk);
    }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    qk = wave_sum(qk);
    const float inv_q = q_scale / sqrtf(sq + unit_eps), inv_k = 1.0f / sqrtf(sk + unit_eps);
    for (int j = lane; j < d; j += WAVE) {
      out[(size_t)g * d + j] = ld(x + (size_t)g * d + j) * inv_q;
      out[(size_t)(groups + g) * d + j] = ld(x + (size_t)(groups + g) * d + j) * inv_k;
    }
    if (lane == 0) out[2 * groups * d + heads + g] = qk * inv_q * inv_k;
  }
  float* zt = z + (size_t)t * heads * d;
  for (int i = tid; i < heads * d; i += 4 * WAVE) zt[i] = expf(neg_rate[i / d] * dl_softplus(zt[i]));
  for (int h = tid; h < heads; h += 4 * WAVE)
    out[2 * groups * d + h] = 1.0f / (1.0f + expf(-ld(beta_rows + (size_t)t * beta_stride + beta_offset + h)));
}

// One workgroup of four waves per (portion, head, 16 columns of S).  A wave owns four columns; its lanes are (column,
// part p = lane % 16): lane (c, p) keeps rows p PER .. p PER + PER - 1 of column c in registers.  Columns of S do not
// depend on each other: for column c, with s = g * S[:, c] (row by row), a = k . s and b = q . s (sums within a row of
// sixteen lanes), u = beta (v_c - a), the new column is s + k u and its read-out q . (s + k u) = b + (q . k) u.
// The rows of q, k (made unit vectors here; q times d^(-1/2)) and of the decays g = exp(neg_rate * softplus(z)) come
// into LDS sixteen tokens at a time; the next sixteen are asked for before the current ones are worked on.
// fresh: rows of `fresh_stride`, [groups d (q) | groups d (k) | heads dv (v)]; z: float rows [heads d]; beta's
// pre-activation at beta_rows[t, beta_offset + h].  A portion that starts at position 0 starts from zeros.
// PREPARED: `delta_prepare_kernel` has run; z holds the decays themselves and `prep` the unit vectors, beta and q . k,
// so that between the trips to memory a workgroup does nothing but the recurrence (long portions: the chain from token
// to token is what bounds them).
template <typename T, int PER, bool PREPARED>
__global__ void __launch_bounds__(4 * WAVE)
delta_scan_kernel(const T* __restrict__ fresh, int fresh_stride, const float* __restrict__ z, const float* __restrict__ neg_rate,
                  const float* __restrict__ prep, const T* __restrict__ beta_rows, int beta_stride, int beta_offset,
                  float* __restrict__ state,
                  size_t state_stride, const int* __restrict__ cu_q, const int* __restrict__ first_position,
                  const int* __restrict__ state_slots, float* __restrict__ out, int heads, int groups, int d, int dv,
                  float unit_eps) {
  constexpr int DP = 16 * PER;                     // rows of S a workgroup's lanes cover (d filled up with zeros)
  constexpr int PIECES = (DL_GROUP * DP) / (4 * WAVE);       // (token, row) pairs a thread brings: PER
  __shared__ __attribute__((aligned(16))) float q_s[DL_GROUP][DP], k_s[DL_GROUP][DP], g_s[DL_GROUP][DP];
  __shared__ float v_s[DL_GROUP][16], beta_s[DL_GROUP], qk_s[DL_GROUP];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int lo = cu_q[e], hi = cu_q[e + 1];
  if (hi <= lo) return;
  const int part = lane & 15, local = wave * 4 + (lane >> 4);
  const int c = blockIdx.z * 16 + local;
  const bool live = c < dv;
  const int qk_head = h / (heads / groups);
  float* mem = state + (size_t)state_slots[e] * state_stride + (size_t)h * d * dv;
  const bool from_zero = first_position[e] == 0;
  float S[PER];
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = part * PER + r;
    S[r] = (!from_zero && live && j < d) ? mem[(size_t)j * dv + c] : 0.f;
  }
  const float rate = PREPARED ? 0.f : neg_rate[h], q_scale = 1.0f / sqrtf((float)d);
  const int prep_width = 2 * groups * d + heads + groups;
  float q_next[PIECES], k_next[PIECES], g_next[PIECES], v_next = 0.f, beta_next = 0.f, qk_next = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int idx = i * 4 * WAVE + tid, tok = idx / DP, j = idx % DP;
      q_next[i] = k_next[i] = 0.f;
      g_next[i] = 0.f;                               // (a pre-activation; rows past d and tokens past the end get decay 1 below)
      if (j < d && t0 + tok < hi) {
        if constexpr (PREPARED) {
          const float* x = prep + (size_t)(t0 + tok) * prep_width;
          q_next[i] = x[(size_t)qk_head * d + j];
          k_next[i] = x[(size_t)(groups + qk_head) * d + j];
        } else {
          const T* x = fresh + (size_t)(t0 + tok) * fresh_stride;
          q_next[i] = ld(x + (size_t)qk_head * d + j);
          k_next[i] = ld(x + (size_t)(groups + qk_head) * d + j);
        }
        g_next[i] = z[(size_t)(t0 + tok) * heads * d + (size_t)h * d + j];
      }
    }
    {
      const int tok = tid >> 4, col = blockIdx.z * 16 + (tid & 15);
      v_next = (col < dv && t0 + tok < hi)
          ? ld(fresh + (size_t)(t0 + tok) * fresh_stride + (size_t)2 * groups * d + (size_t)h * dv + col) : 0.f;
    }
    if constexpr (PREPARED) {
      if (tid < DL_GROUP && t0 + tid < hi) {
        const float* x = prep + (size_t)(t0 + tid) * prep_width + 2 * groups * d;
        beta_next = x[h];
        qk_next = x[heads + qk_head];
      }
    } else {
      if (tid < DL_GROUP) beta_next = t0 + tid < hi ? ld(beta_rows + (size_t)(t0 + tid) * beta_stride + beta_offset + h) : 0.f;
    }
  };
  fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += DL_GROUP) {
    __syncthreads();                                         // the group before has been worked off
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int idx = i * 4 * WAVE + tid, tok = idx / DP, j = idx % DP;
      q_s[tok][j] = q_next[i];
      k_s[tok][j] = k_next[i];
      if constexpr (PREPARED) g_s[tok][j] = (j < d && t0 + tok < hi) ? g_next[i] : 1.f;
      else g_s[tok][j] = (j < d && t0 + tok < hi) ? expf(rate * dl_softplus(g_next[i])) : 1.f;
    }
    v_s[tid >> 4][tid & 15] = v_next;
    if constexpr (PREPARED) {
      if (tid < DL_GROUP) {
        beta_s[tid] = t0 + tid < hi ? beta_next : 0.f;
        qk_s[tid] = t0 + tid < hi ? qk_next : 0.f;
      }
    } else {
      if (tid < DL_GROUP) beta_s[tid] = t0 + tid < hi ? 1.0f / (1.0f + expf(-beta_next)) : 0.f;
    }
    if (t0 + DL_GROUP < hi) fetch(t0 + DL_GROUP);
    __syncthreads();
    // Unit vectors: sixteen threads a token add up the squares (and q . k) over the rows, then scale the rows in place.
    if constexpr (!PREPARED) {
      const int tok = tid >> 4, p = tid & 15;
      float sq = 0.f, sk = 0.f, qk = 0.f;
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        const float qv = q_s[tok][p + 16 * r], kv = k_s[tok][p + 16 * r];
        sq = fmaf(qv, qv, sq);
        sk = fmaf(kv, kv, sk);
        qk = fmaf(qv, kv, qk);
      }
      sq = dl_row_sum16(sq);
      sk = dl_row_sum16(sk);
      qk = dl_row_sum16(qk);
      const float inv_q = q_scale / sqrtf(sq + unit_eps), inv_k = 1.0f / sqrtf(sk + unit_eps);
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        q_s[tok][p + 16 * r] *= inv_q;
        k_s[tok][p + 16 * r] *= inv_k;
      }
      if (p == 0) qk_s[tok] = qk * inv_q * inv_k;
      __syncthreads();
    }
    // Token by token.  (A token past the portion's end has decay 1, beta 0 and zeros for q, k and v: it changes nothing.
    // Rows past d hold zeros in q and k and decay 1: they stay zero and add nothing.)
    float read[DL_GROUP];
#pragma unroll
    for (int tok = 0; tok < DL_GROUP; ++tok) {
      float a = 0.f, b = 0.f;
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        S[r] *= g_s[tok][part * PER + r];
        a = fmaf(k_s[tok][part * PER + r], S[r], a);
        b = fmaf(q_s[tok][part * PER + r], S[r], b);
      }
      a = dl_row_sum16(a);
      b = dl_row_sum16(b);
      const float u = beta_s[tok] * (v_s[tok][local] - a);
#pragma unroll
      for (int r = 0; r < PER; ++r) S[r] = fmaf(k_s[tok][part * PER + r], u, S[r]);
      read[tok] = fmaf(qk_s[tok], u, b);
    }
    if (part == 0 && live) {
#pragma unroll
      for (int tok = 0; tok < DL_GROUP; ++tok)
        if (t0 + tok < hi) out[(size_t)(t0 + tok) * heads * dv + (size_t)h * dv + c] = read[tok];
    }
  }
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = part * PER + r;
    if (live && j < d) mem[(size_t)j * dv + c] = S[r];
  }
}

// rows: [n_tokens, row_stride]; the channels are three runs of its columns (offsets o0..o2, widths w0..w2); taps float
// [channels, n_taps]; out [n_tokens, channels].
extern "C" int ta_short_conv_silu(const void* rows, int row_stride, int o0, int w0, int o1, int w1, int o2, int w2,
                                  const void* taps, int n_taps, void* state, long state_stride, int state_offset,
                                  const void* cu_q, const void* first_position, const void* state_slots,
                                  const void* entry_of_token, void* out, int n_tokens, int n_entries, int dtype,
                                  const void* bias, hipStream_t stream) {
  if (n_tokens <= 0 || n_entries <= 0) return 0;
  const int channels = w0 + w1 + w2;
  if (channels <= 0 || w0 < 0 || w1 < 0 || w2 < 0 || n_taps < 1 || n_taps > DL_MAX_TAPS || channels > 65535 * 256 ||
      state_stride < (long)state_offset + (long)(n_taps - 1) * channels)
    return -1;
  ConvRuns runs = {{o0, o1, o2}, {w0, w1, w2}};
  dim3 per_token(n_tokens, (channels + 255) / 256), per_entry(n_entries, (channels + 255) / 256);
#define CONV(TT)                                                                                                           \
  short_conv_silu_kernel<TT><<<per_token, 256, 0, stream>>>((const TT*)rows, row_stride, runs, channels, (const float*)taps, \
      n_taps, (const float*)state, (size_t)state_stride, state_offset, (const int*)cu_q, (const int*)first_position,        \
      (const int*)state_slots, (const int*)entry_of_token, (TT*)out, (const float*)bias);                                  \
  if (n_taps > 1)                                                                                                          \
    short_conv_keep_kernel<TT><<<per_entry, 256, 0, stream>>>((const TT*)rows, row_stride, runs, channels, n_taps,          \
        (float*)state, (size_t)state_stride, state_offset, (const int*)cu_q, (const int*)first_position,                   \
        (const int*)state_slots)
  if (dtype == DT_F32) { CONV(float); } else { CONV(bf16_t); }
#undef CONV
  return LAUNCH_STATUS();
}

// fresh: rows of `fresh_stride` elements, [groups d (q) | groups d (k) | heads dv (v)]; z float [n_tokens, heads d];
// neg_rate float [heads]; out float [n_tokens, heads dv].  prep: null, or room for n_tokens rows of
// 2 groups d + heads + groups floats: then what does not depend on the state is made for all tokens side by side first
// (z then holds the decays afterwards), which is what steps with long portions want.
extern "C" int ta_delta_scan(const void* fresh, int fresh_stride, void* z, const void* neg_rate, const void* beta_rows,
                             int beta_stride, int beta_offset, void* state, long state_stride, const void* cu_q,
                             const void* first_position, const void* state_slots, void* out, void* prep, int n_tokens,
                             int n_entries, int heads, int groups, int d, int dv, float unit_eps, int dtype,
                             hipStream_t stream) {
  if (n_entries <= 0 || n_tokens <= 0) return 0;
  if (d < 1 || d > DL_MAX_D || dv < 1 || heads < 1 || groups < 1 || heads % groups || heads > 65535 ||
      state_stride < (long)heads * d * dv)
    return -1;
  dim3 grid(n_entries, heads, (dv + 15) / 16);
  if (grid.z > 65535) return -1;
  const int per = (d + 15) / 16;
  if (prep) {
    if (dtype == DT_F32)
      delta_prepare_kernel<float><<<n_tokens, 4 * WAVE, 0, stream>>>((const float*)fresh, fresh_stride, (float*)z,
          (const float*)neg_rate, (const float*)beta_rows, beta_stride, beta_offset, (float*)prep, heads, groups, d, unit_eps);
    else
      delta_prepare_kernel<bf16_t><<<n_tokens, 4 * WAVE, 0, stream>>>((const bf16_t*)fresh, fresh_stride, (float*)z,
          (const float*)neg_rate, (const bf16_t*)beta_rows, beta_stride, beta_offset, (float*)prep, heads, groups, d, unit_eps);
  }
#define SCAN(TT, PP, RR) delta_scan_kernel<TT, PP, RR><<<grid, 4 * WAVE, 0, stream>>>((const TT*)fresh, fresh_stride,        \
    (const float*)z, (const float*)neg_rate, (const float*)prep, (const TT*)beta_rows, beta_stride, beta_offset,             \
    (float*)state, (size_t)state_stride, (const int*)cu_q, (const int*)first_position, (const int*)state_slots,             \
    (float*)out, heads, groups, d, dv, unit_eps)
#define SCANS(TT, RR) if (per <= 1) SCAN(TT, 1, RR); else if (per <= 2) SCAN(TT, 2, RR); else if (per <= 4) SCAN(TT, 4, RR); \
                      else if (per <= 8) SCAN(TT, 8, RR); else SCAN(TT, 16, RR)
  if (prep) {
    if (dtype == DT_F32) { SCANS(float, true); } else { SCANS(bf16_t, true); }
  } else {
    if (dtype == DT_F32) { SCANS(float, false); } else { SCANS(bf16_t, false); }
  }
#undef SCANS
#undef SCAN
  return LAUNCH_STATUS();
}
