// Routed feed-forwards and the per-layer token input: the choice of experts from float router logits, the gated
// activation of the chosen experts with their weights folded in, and the gate of the token input.
#include "common.h"

__device__ __forceinline__ float rt_gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// logits: float [n_tokens, n_experts].  For every token the `top` largest logits (the lower index of equals) in falling
// order: chosen [n_tokens, top] and weights [n_tokens, top] = softmax over those logits alone.  A wave a token.
__global__ void __launch_bounds__(256)
route_top_kernel(const float* __restrict__ logits, int n_tokens, int n_experts, int top, int* __restrict__ chosen,
                 float* __restrict__ weights) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int t = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (t >= n_tokens) return;
  const float* row = logits + (size_t)t * n_experts;
  float top_value = 0.f, total = 0.f, mine = 0.f;
  int last = -1;
  float last_value = INFINITY;
  for (int k = 0; k < top; ++k) {
    // The largest logit that comes behind the one picked last in the order (value falling, index rising).
    float best = -INFINITY;
    int best_at = n_experts;
    for (int e = lane; e < n_experts; e += WAVE) {
      const float v = row[e];
      const bool behind = v < last_value || (v == last_value && e > last);
      if (behind && (v > best || (v == best && e < best_at))) { best = v; best_at = e; }
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, WAVE);
      const int other_at = __shfl_xor(best_at, off, WAVE);
      if (other > best || (other == best && other_at < best_at)) { best = other; best_at = other_at; }
    }
    if (k == 0) top_value = best;
    const float e = expf(best - top_value);
    total += e;
    if (lane == k) mine = e;                        // lane k keeps pick k's term
    if (lane == 0) chosen[(size_t)t * top + k] = best_at;
    last = best_at;
    last_value = best;
  }
  // Every lane holds the same total, lane k pick k's term (the launcher takes top <= 64).
  if (lane < top) weights[(size_t)t * top + lane] = mine / total;
}

// Eight bfloat16 elements (sixteen bytes) as floats, and back.
__device__ __forceinline__ void rt_unpack8(const uint4 raw, float (&v)[8]) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(w[i] << 16); v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
}
__device__ __forceinline__ uint4 rt_pack8(const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = (uint32_t)float_to_bf16_bits(v[2 * i]) | ((uint32_t)float_to_bf16_bits(v[2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

#define RT_MAX_EXPERTS 256
#define RT_ROW_PIECES 8        // sixteen-byte pieces of a row that a lane keeps: rows of up to 64 * 8 * 8 bfloat16 elements

template <typename T> struct RtVec;
template <> struct RtVec<bf16_t> {
  static constexpr int N = 8;
  __device__ static __forceinline__ void load(const bf16_t* p, float (&v)[8]) { rt_unpack8(*reinterpret_cast<const uint4*>(p), v); }
};
template <> struct RtVec<float> {
  static constexpr int N = 4;
  __device__ static __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 raw = *reinterpret_cast<const float4*>(p);
    v[0] = raw.x; v[1] = raw.y; v[2] = raw.z; v[3] = raw.w;
  }
};

// The router's product and the choice in one kernel, a workgroup a token: x [n_tokens, hidden] (row stride lda) and
// router [n_experts, hidden] of type T in pieces of sixteen bytes; wave w forms the logits of experts w, w + 4, ... as
// float sums (a lane keeps its pieces of the row), wave 0 then picks as route_top_kernel does.
template <typename T>
__global__ void __launch_bounds__(256)
route_rows_kernel(const T* __restrict__ x, int lda, const T* __restrict__ router, int hidden, int n_experts, int top,
                  int* __restrict__ chosen, float* __restrict__ weights) {
  constexpr int N = RtVec<T>::N;
  __shared__ float logit_s[RT_MAX_EXPERTS];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const T* row = x + (size_t)t * lda;
  float xv[RT_ROW_PIECES][N];
#pragma unroll
  for (int p = 0; p < RT_ROW_PIECES; ++p) {
    const int at = (p * WAVE + lane) * N;
    if (at < hidden) RtVec<T>::load(row + at, xv[p]);
    else
#pragma unroll
      for (int k = 0; k < N; ++k) xv[p][k] = 0.f;
  }
  for (int e = wave; e < n_experts; e += 256 / WAVE) {
    const T* w = router + (size_t)e * hidden;
    float sum = 0.f;
#pragma unroll
    for (int p = 0; p < RT_ROW_PIECES; ++p) {
      const int at = (p * WAVE + lane) * N;
      if (at < hidden) {
        float wv[N];
        RtVec<T>::load(w + at, wv);
#pragma unroll
        for (int k = 0; k < N; ++k) sum = fmaf(wv[k], xv[p][k], sum);
      }
    }
    sum = wave_sum(sum);
    if (lane == 0) logit_s[e] = sum;
  }
  __syncthreads();
  if (wave != 0) return;
  float top_value = 0.f, total = 0.f, mine = 0.f, last_value = INFINITY;
  int last = -1;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int best_at = n_experts;
    for (int e = lane; e < n_experts; e += WAVE) {
      const float v = logit_s[e];
      const bool behind = v < last_value || (v == last_value && e > last);
      if (behind && (v > best || (v == best && e < best_at))) { best = v; best_at = e; }
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, WAVE);
      const int other_at = __shfl_xor(best_at, off, WAVE);
      if (other > best || (other == best && other_at < best_at)) { best = other; best_at = other_at; }
    }
    if (k == 0) top_value = best;
    const float term = expf(best - top_value);
    total += term;
    if (lane == k) mine = term;
    if (lane == 0) chosen[(size_t)t * top + k] = best_at;
    last = best_at;
    last_value = best;
  }
  if (lane < top) weights[(size_t)t * top + lane] = mine / total;
}

// gate_up: [n_tokens, n_experts * 2 * inner + 2 * shared], expert e's gate rows then its up rows, the shared expert
// last.  out: [n_tokens, columns] with columns >= n_experts * inner + shared: out[t, e * inner + i] =
// w * silu(gate) * up for an expert the token chose with weight w, 0 for the others; the shared expert's columns
// with weight 1 (or shared_weight[t], float, where given); columns beyond are 0.
template <typename T>
__global__ void expert_gate_kernel(const T* __restrict__ gate_up, const int* __restrict__ chosen,
                                   const float* __restrict__ weights, int top, int n_experts, int inner, int shared,
                                   int columns, T* __restrict__ out, size_t total, const float* __restrict__ shared_weight) {
  const int in_stride = n_experts * 2 * inner + 2 * shared;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / columns;
    const int c = (int)(idx - t * columns);
    const T* row = gate_up + t * in_stride;
    float value = 0.f;
    if (c < n_experts * inner) {
      const int e = c / inner, i = c - e * inner;
      float w = 0.f;
      for (int k = 0; k < top; ++k)
        if (chosen[t * top + k] == e) w += weights[t * top + k];
      if (w != 0.f) {
        const float g = ld(row + (size_t)e * 2 * inner + i), u = ld(row + (size_t)e * 2 * inner + inner + i);
        value = w * (g / (1.0f + expf(-g)) * u);
      }
    } else if (c < n_experts * inner + shared) {
      const int i = c - n_experts * inner;
      const float g = ld(row + (size_t)n_experts * 2 * inner + i), u = ld(row + (size_t)n_experts * 2 * inner + shared + i);
      value = g / (1.0f + expf(-g)) * u;
      if (shared_weight) value *= shared_weight[t];
    }
    st(out + idx, value);
  }
}

// out[t, j] = gelu_tanh(gate[t, j]) * table[token_ids[t], offset + j] for j < dim, 0 for dim <= j < columns.
// gate, out: [n_tokens, columns]; table: [vocab, table_width].
template <typename T>
__global__ void side_gate_kernel(const T* __restrict__ gate, const T* __restrict__ table, int table_width,
                                 const int* __restrict__ token_ids, int offset, int dim, int columns,
                                 T* __restrict__ out, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / columns;
    const int j = (int)(idx - t * columns);
    float value = 0.f;
    if (j < dim) value = rt_gelu_tanh(ld(gate + idx)) * ld(table + (size_t)token_ids[t] * table_width + offset + j);
    st(out + idx, value);
  }
}

// out[t, j] = gelu_tanh(in[t, j]) * in[t, inner + j].
template <typename T>
__global__ void gelu_gate_kernel(const T* __restrict__ in, T* __restrict__ out, int inner, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inner;
    const int j = (int)(idx - t * inner);
    st(out + idx, rt_gelu_tanh(ld(in + t * 2 * inner + j)) * ld(in + t * 2 * inner + inner + j));
  }
}

// expert_gate for bfloat16 with inner, shared and columns multiples of 8: a thread makes eight columns, which lie in
// one expert; the rows of experts a token did not choose are not read.
__global__ void expert_gate_vec_kernel(const bf16_t* __restrict__ gate_up, const int* __restrict__ chosen,
                                       const float* __restrict__ weights, int top, int n_experts, int inner, int shared,
                                       int columns, bf16_t* __restrict__ out, size_t total8,
                                       const float* __restrict__ shared_weight) {
  const int in_stride = n_experts * 2 * inner + 2 * shared, columns8 = columns / 8;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total8; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / columns8;
    const int c = (int)(idx - t * columns8) * 8;
    const bf16_t* row = gate_up + t * in_stride;
    const bf16_t* g_at = nullptr;
    int up_off = 0;
    float w = 0.f;
    if (c < n_experts * inner) {
      const int e = c / inner, i = c - e * inner;
      for (int k = 0; k < top; ++k)
        if (chosen[t * top + k] == e) w += weights[t * top + k];
      if (w != 0.f) { g_at = row + (size_t)e * 2 * inner + i; up_off = inner; }
    } else if (c < n_experts * inner + shared) {
      g_at = row + (size_t)n_experts * 2 * inner + (c - n_experts * inner);
      up_off = shared;
      w = shared_weight ? shared_weight[t] : 1.f;
    }
    uint4 packed = make_uint4(0, 0, 0, 0);
    if (g_at) {
      float g[8], u[8], v[8];
      rt_unpack8(*reinterpret_cast<const uint4*>(g_at), g);
      rt_unpack8(*reinterpret_cast<const uint4*>(g_at + up_off), u);
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = w * (g[k] / (1.0f + expf(-g[k])) * u[k]);
      packed = rt_pack8(v);
    }
    *reinterpret_cast<uint4*>(out + t * columns + c) = packed;
  }
}

// gelu_gate for bfloat16 rows whose length is a multiple of 8: sixteen bytes of gate and of up per thread.
__global__ void gelu_gate_vec_kernel(const bf16_t* __restrict__ in, bf16_t* __restrict__ out, int inner8, size_t total8) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total8; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / inner8, j = idx - t * inner8;
    const uint4* row = reinterpret_cast<const uint4*>(in) + t * 2 * inner8;
    float g[8], u[8], v[8];
    rt_unpack8(row[j], g);
    rt_unpack8(row[inner8 + j], u);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = rt_gelu_tanh(g[k]) * u[k];
    reinterpret_cast<uint4*>(out)[idx] = rt_pack8(v);
  }
}

static inline int rt_blocks(size_t total) { return (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535); }

extern "C" int ta_route_top(const void* logits, int n_tokens, int n_experts, int top, void* chosen, void* weights,
                            hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (top <= 0 || top > n_experts || top > WAVE) return -1;
  route_top_kernel<<<(n_tokens + 3) / 4, 256, 0, stream>>>((const float*)logits, n_tokens, n_experts, top, (int*)chosen,
                                                           (float*)weights);
  return LAUNCH_STATUS();
}

// Returns -2 for sizes the fused kernel does not take (the caller then forms the logits with a product of its own).
extern "C" int ta_route_rows(const void* x, int lda, const void* router, int n_tokens, int hidden, int n_experts, int top,
                             void* chosen, void* weights, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (top <= 0 || top > n_experts || top > WAVE) return -1;
  const int piece = dtype == DT_F32 ? 4 : 8;
  if (n_experts > RT_MAX_EXPERTS || hidden % piece || lda % piece || hidden > WAVE * RT_ROW_PIECES * piece ||
      (((uintptr_t)x | (uintptr_t)router) & 15))
    return -2;
  if (dtype == DT_F32)
    route_rows_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)x, lda, (const float*)router, hidden, n_experts, top,
                                                           (int*)chosen, (float*)weights);
  else
    route_rows_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)x, lda, (const bf16_t*)router, hidden, n_experts,
                                                            top, (int*)chosen, (float*)weights);
  return LAUNCH_STATUS();
}

extern "C" int ta_expert_gate(const void* gate_up, const void* chosen, const void* weights, int n_tokens, int top,
                              int n_experts, int inner, int shared, int columns, void* out, int dtype,
                              const void* shared_weight, hipStream_t stream) {
  const size_t total = (size_t)n_tokens * columns;
  if (total == 0) return 0;
  if (columns < n_experts * inner + shared) return -1;
  if (dtype == DT_BF16 && inner % 8 == 0 && shared % 8 == 0 && columns % 8 == 0 &&
      (((uintptr_t)gate_up | (uintptr_t)out) & 15) == 0) {
    expert_gate_vec_kernel<<<rt_blocks(total / 8), 256, 0, stream>>>((const bf16_t*)gate_up, (const int*)chosen,
        (const float*)weights, top, n_experts, inner, shared, columns, (bf16_t*)out, total / 8, (const float*)shared_weight);
    return LAUNCH_STATUS();
  }
  if (dtype == DT_F32)
    expert_gate_kernel<float><<<rt_blocks(total), 256, 0, stream>>>((const float*)gate_up, (const int*)chosen,
        (const float*)weights, top, n_experts, inner, shared, columns, (float*)out, total, (const float*)shared_weight);
  else
    expert_gate_kernel<bf16_t><<<rt_blocks(total), 256, 0, stream>>>((const bf16_t*)gate_up, (const int*)chosen,
        (const float*)weights, top, n_experts, inner, shared, columns, (bf16_t*)out, total, (const float*)shared_weight);
  return LAUNCH_STATUS();
}

extern "C" int ta_side_gate(const void* gate, const void* table, int table_width, const void* token_ids, int offset, int dim,
                            int columns, int n_tokens, void* out, int dtype, hipStream_t stream) {
  const size_t total = (size_t)n_tokens * columns;
  if (total == 0) return 0;
  if (dim > columns || offset < 0 || offset + dim > table_width) return -1;
  if (dtype == DT_F32)
    side_gate_kernel<float><<<rt_blocks(total), 256, 0, stream>>>((const float*)gate, (const float*)table, table_width,
        (const int*)token_ids, offset, dim, columns, (float*)out, total);
  else
    side_gate_kernel<bf16_t><<<rt_blocks(total), 256, 0, stream>>>((const bf16_t*)gate, (const bf16_t*)table, table_width,
        (const int*)token_ids, offset, dim, columns, (bf16_t*)out, total);
  return LAUNCH_STATUS();
}

extern "C" int ta_gelu_gate(const void* in, void* out, int n_tokens, int inner, int dtype, hipStream_t stream) {
  const size_t total = (size_t)n_tokens * inner;
  if (total == 0) return 0;
  if (dtype == DT_BF16 && inner % 8 == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0) {
    gelu_gate_vec_kernel<<<rt_blocks(total / 8), 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, inner / 8, total / 8);
    return LAUNCH_STATUS();
  }
  if (dtype == DT_F32)
    gelu_gate_kernel<float><<<rt_blocks(total), 256, 0, stream>>>((const float*)in, (float*)out, inner, total);
  else
    gelu_gate_kernel<bf16_t><<<rt_blocks(total), 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, inner, total);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------------------------------
// A router of sigmoid scores with a correction and groups, and experts without a gate branch.

#define RS_MAX_EXPERTS 1024

// logits: float [n_tokens, n_experts].  s = sigmoid(logit); an expert's choice score is s + correction.  With n_groups > 0
// the experts form that many equal groups of neighbours; a group is worth the sum of its two largest choice scores (its
// one score if it has one expert), and experts outside the `keep` best groups (the lower index of equals) count as minus
// infinity.  The `top` largest choice scores (the lower index of equals) are chosen, in falling order; their weights
// are their s over the sum of the chosen s (+ 1e-20).  A wave a token; the scores of a token lie in LDS.
// The choice among one token's scores in LDS (`choice`: s + correction, `score`: s, `worth`: room for a number a group).
// Every wave that calls it for a token runs the same steps between the same barriers (waves that share a token write
// the same values); `store` says whether this wave writes the token's results.
__device__ __forceinline__ void rs_choose(float* choice, const float* score, float* worth, int lane, int n_experts,
                                          int n_groups, int keep, int top, bool store, int* __restrict__ chosen_row,
                                          float* __restrict__ weights_row, bool group_max = false) {
  if (n_groups > 0) {
    const int per = n_experts / n_groups;
    for (int g = lane; g < n_groups; g += WAVE) {
      float first = -INFINITY, second = -INFINITY;
      for (int i = 0; i < per; ++i) {
        const float v = choice[g * per + i];
        if (v > first) { second = first; first = v; }
        else if (v > second) second = v;
      }
      worth[g] = (per > 1 && !group_max) ? first + second : first;
    }
    __syncthreads();
    for (int g = lane; g < n_groups; g += WAVE) {
      const float mine = worth[g];
      int ahead = 0;
      for (int o = 0; o < n_groups; ++o) {
        const float v = worth[o];
        ahead += (v > mine || (v == mine && o < g)) ? 1 : 0;
      }
      if (ahead >= keep)
        for (int i = 0; i < per; ++i) choice[g * per + i] = -INFINITY;
    }
    __syncthreads();
  }
  float total = 0.f, mine = 0.f;
  int last = -1;
  float last_value = INFINITY;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int best_at = n_experts;
    for (int e = lane; e < n_experts; e += WAVE) {
      const float v = choice[e];
      const bool behind = v < last_value || (v == last_value && e > last);
      if (behind && (v > best || (v == best && e < best_at))) { best = v; best_at = e; }
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, WAVE);
      const int other_at = __shfl_xor(best_at, off, WAVE);
      if (other > best || (other == best && other_at < best_at)) { best = other; best_at = other_at; }
    }
    best_at = min(best_at, n_experts - 1);
    const float s = score[best_at];
    total += s;
    if (lane == k) mine = s;
    if (store && lane == 0) chosen_row[k] = best_at;
    last = best_at;
    last_value = best;
  }
  if (store && lane < top) weights_row[lane] = mine / (total + 1e-20f);
}

__global__ void __launch_bounds__(256)
route_sigmoid_kernel(const float* __restrict__ logits, const float* __restrict__ correction, int n_tokens, int n_experts,
                     int n_groups, int keep, int top, int* __restrict__ chosen, float* __restrict__ weights) {
  extern __shared__ float rs_scratch[];
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int slot = blockIdx.x * (blockDim.x / WAVE) + wave;
  const bool live = slot < n_tokens;                          // (a wave past the end works on the last token and stores nothing)
  const int t = live ? slot : n_tokens - 1;
  float* choice = rs_scratch + (size_t)wave * (2 * n_experts + n_groups);
  float* score = choice + n_experts;
  float* worth = score + n_experts;
  const float* row = logits + (size_t)t * n_experts;
  for (int e = lane; e < n_experts; e += WAVE) {
    const float s = 1.0f / (1.0f + expf(-row[e]));
    score[e] = s;
    choice[e] = s + correction[e];
  }
  __syncthreads();
  rs_choose(choice, score, worth, lane, n_experts, n_groups, keep, top, live, chosen + (size_t)t * top, weights + (size_t)t * top);
}

// The same choice from scores of either kind.  logits: float rows of `stride` numbers, the experts' first.  softmax: the
// scores are the softmax over all experts (else sigmoid); correction may be null; group_max: a group is worth its
// largest choice score (else the sum of its two largest); gate (float [n_tokens] or null) gets sigmoid of the number
// behind the experts' logits in the row.  A wave a token.
__global__ void __launch_bounds__(256)
route_scores_kernel(const float* __restrict__ logits, int stride, const float* __restrict__ correction, int n_tokens,
                    int n_experts, int n_groups, int keep, int top, int softmax, int group_max, int* __restrict__ chosen,
                    float* __restrict__ weights, float* __restrict__ gate) {
  extern __shared__ float rs_scratch[];
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int slot = blockIdx.x * (blockDim.x / WAVE) + wave;
  const bool live = slot < n_tokens;                          // (a wave past the end works on the last token and stores nothing)
  const int t = live ? slot : n_tokens - 1;
  float* choice = rs_scratch + (size_t)wave * (2 * n_experts + n_groups);
  float* score = choice + n_experts;
  float* worth = score + n_experts;
  const float* row = logits + (size_t)t * stride;
  float top_logit = -INFINITY, total = 1.f;
  if (softmax) {
    for (int e = lane; e < n_experts; e += WAVE) top_logit = fmaxf(top_logit, row[e]);
    top_logit = wave_max(top_logit);
    total = 0.f;
    for (int e = lane; e < n_experts; e += WAVE) total += expf(row[e] - top_logit);
    total = wave_sum(total);
  }
  for (int e = lane; e < n_experts; e += WAVE) {
    const float s = softmax ? expf(row[e] - top_logit) / total : 1.0f / (1.0f + expf(-row[e]));
    score[e] = s;
    choice[e] = correction ? s + correction[e] : s;
  }
  if (gate && live && lane == 0) gate[t] = 1.0f / (1.0f + expf(-row[n_experts]));
  __syncthreads();
  rs_choose(choice, score, worth, lane, n_experts, n_groups, keep, top, live, chosen + (size_t)t * top,
            weights + (size_t)t * top, group_max != 0);
}

// The router's product and the choice in one kernel, a token a workgroup (few rows: a decode step): as route_rows_kernel
// forms the logits (float sums of the row with each expert's router row, the row kept in registers), then all four
// waves choose together and the first stores.
template <typename T>
__global__ void __launch_bounds__(256)
route_rows_sigmoid_kernel(const T* __restrict__ x, int lda, const T* __restrict__ router, const float* __restrict__ correction,
                          int hidden, int n_experts, int n_groups, int keep, int top, int* __restrict__ chosen,
                          float* __restrict__ weights, int softmax = 0, int group_max = 0, float* __restrict__ gate = nullptr) {
  constexpr int N = RtVec<T>::N;
  extern __shared__ float rs_scratch[];
  float* choice = rs_scratch;
  float* score = choice + n_experts;
  float* worth = score + n_experts;
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const T* row = x + (size_t)t * lda;
  float xv[RT_ROW_PIECES][N];
#pragma unroll
  for (int p = 0; p < RT_ROW_PIECES; ++p) {
    const int at = (p * WAVE + lane) * N;
    if (at < hidden) RtVec<T>::load(row + at, xv[p]);
    else
#pragma unroll
      for (int k = 0; k < N; ++k) xv[p][k] = 0.f;
  }
  // (With a gate, the router has one row more: the gate's, behind the experts'.)
  for (int e = wave; e < n_experts + (gate ? 1 : 0); e += 256 / WAVE) {
    const T* w = router + (size_t)e * hidden;
    float sum = 0.f;
#pragma unroll
    for (int p = 0; p < RT_ROW_PIECES; ++p) {
      const int at = (p * WAVE + lane) * N;
      if (at < hidden) {
        float wv[N];
        RtVec<T>::load(w + at, wv);
#pragma unroll
        for (int k = 0; k < N; ++k) sum = fmaf(wv[k], xv[p][k], sum);
      }
    }
    sum = wave_sum(sum);
    if (lane == 0) {
      if (e == n_experts) {
        gate[t] = 1.0f / (1.0f + expf(-sum));
      } else if (softmax) {
        score[e] = sum;                                      // the logit, until all of them are there
      } else {
        const float s = 1.0f / (1.0f + expf(-sum));
        score[e] = s;
        choice[e] = correction ? s + correction[e] : s;
      }
    }
  }
  __syncthreads();
  if (softmax) {                                             // every thread sums the few logits up for itself
    float top_logit = -INFINITY, total = 0.f;
    for (int e = 0; e < n_experts; ++e) top_logit = fmaxf(top_logit, score[e]);
    for (int e = 0; e < n_experts; ++e) total += expf(score[e] - top_logit);
    __syncthreads();
    for (int e = threadIdx.x; e < n_experts; e += 256) {
      const float s = expf(score[e] - top_logit) / total;
      score[e] = s;
      choice[e] = correction ? s + correction[e] : s;
    }
    __syncthreads();
  }
  rs_choose(choice, score, worth, lane, n_experts, n_groups, keep, top, wave == 0, chosen + (size_t)t * top,
            weights + (size_t)t * top, group_max != 0);
}

// up: [n_tokens, n_experts * inner]; out: [n_tokens, columns], columns >= n_experts * inner:
// out[t, e * inner + i] = w * max(up, 0)^2 for an expert the token chose with weight w, 0 for the others and beyond.
template <typename T>
__global__ void expert_act_kernel(const T* __restrict__ up, const int* __restrict__ chosen, const float* __restrict__ weights,
                                  int top, int n_experts, int inner, int columns, T* __restrict__ out, size_t total) {
  const int in_stride = n_experts * inner;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / columns;
    const int c = (int)(idx - t * columns);
    float value = 0.f;
    if (c < in_stride) {
      const int e = c / inner;
      float w = 0.f;
      for (int k = 0; k < top; ++k)
        if (chosen[t * top + k] == e) w += weights[t * top + k];
      if (w != 0.f) {
        const float z = fmaxf(ld(up + t * in_stride + c), 0.f);
        value = w * (z * z);
      }
    }
    st(out + idx, value);
  }
}

// The same for bfloat16 rows in pieces of eight (inner and columns multiples of eight).
__global__ void expert_act_vec_kernel(const bf16_t* __restrict__ up, const int* __restrict__ chosen,
                                      const float* __restrict__ weights, int top, int n_experts, int inner, int columns,
                                      bf16_t* __restrict__ out, size_t total8) {
  const int in_stride = n_experts * inner, columns8 = columns / 8;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total8; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / columns8;
    const int c = (int)(idx - t * columns8) * 8;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (c < in_stride) {
      const int e = c / inner;
      float w = 0.f;
      for (int k = 0; k < top; ++k)
        if (chosen[t * top + k] == e) w += weights[t * top + k];
      if (w != 0.f) {
        rt_unpack8(*reinterpret_cast<const uint4*>(up + t * in_stride + c), v);
#pragma unroll
        for (int i = 0; i < 8; ++i) { const float z = fmaxf(v[i], 0.f); v[i] = w * (z * z); }
      }
    }
    *reinterpret_cast<uint4*>(out + idx * 8) = rt_pack8(v);
  }
}

// out = max(in, 0)^2, element by element.
template <typename T>
__global__ void relu2_kernel(const T* __restrict__ in, T* __restrict__ out, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const float z = fmaxf(ld(in + idx), 0.f);
    st(out + idx, z * z);
  }
}

__global__ void relu2_vec_kernel(const bf16_t* __restrict__ in, bf16_t* __restrict__ out, size_t total8) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total8; idx += (size_t)gridDim.x * blockDim.x) {
    float v[8];
    rt_unpack8(*reinterpret_cast<const uint4*>(in + idx * 8), v);
#pragma unroll
    for (int i = 0; i < 8; ++i) { const float z = fmaxf(v[i], 0.f); v[i] = z * z; }
    *reinterpret_cast<uint4*>(out + idx * 8) = rt_pack8(v);
  }
}

extern "C" int ta_route_sigmoid(const void* logits, const void* correction, int n_tokens, int n_experts, int n_groups,
                                int keep, int top, void* chosen, void* weights, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (top <= 0 || top > n_experts || top > WAVE || n_experts > RS_MAX_EXPERTS || n_groups < 0) return -1;
  if (n_groups > 0 && (n_experts % n_groups || keep <= 0 || keep > n_groups || keep * (n_experts / n_groups) < top)) return -1;
  const size_t lds = (size_t)4 * (2 * n_experts + n_groups) * sizeof(float);
  route_sigmoid_kernel<<<(n_tokens + 3) / 4, 256, lds, stream>>>((const float*)logits, (const float*)correction, n_tokens,
                                                                 n_experts, n_groups, keep, top, (int*)chosen, (float*)weights);
  return LAUNCH_STATUS();
}

extern "C" int ta_route_scores(const void* logits, int stride, const void* correction, int n_tokens, int n_experts,
                               int n_groups, int keep, int top, int softmax, int group_max, void* chosen, void* weights,
                               void* gate, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (top <= 0 || top > n_experts || top > WAVE || n_experts > RS_MAX_EXPERTS || n_groups < 0) return -1;
  if (stride < n_experts + (gate ? 1 : 0)) return -1;
  if (n_groups > 0 && (n_experts % n_groups || keep <= 0 || keep > n_groups || keep * (n_experts / n_groups) < top)) return -1;
  const size_t lds = (size_t)4 * (2 * n_experts + n_groups) * sizeof(float);
  route_scores_kernel<<<(n_tokens + 3) / 4, 256, lds, stream>>>((const float*)logits, stride, (const float*)correction,
      n_tokens, n_experts, n_groups, keep, top, softmax, group_max, (int*)chosen, (float*)weights, (float*)gate);
  return LAUNCH_STATUS();
}

// The same for scores of either kind (see route_scores_kernel): router [n_experts (+ 1 with a gate), hidden].
extern "C" int ta_route_rows_scores(const void* x, int lda, const void* router, const void* correction, int n_tokens,
                                    int hidden, int n_experts, int n_groups, int keep, int top, int softmax, int group_max,
                                    void* chosen, void* weights, void* gate, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (top <= 0 || top > n_experts || top > WAVE || n_groups < 0) return -1;
  if (n_groups > 0 && (n_experts % n_groups || keep <= 0 || keep > n_groups || keep * (n_experts / n_groups) < top)) return -1;
  const int piece = dtype == DT_F32 ? 4 : 8;
  if (n_experts > RT_MAX_EXPERTS || hidden % piece || lda % piece || hidden > WAVE * RT_ROW_PIECES * piece ||
      (((uintptr_t)x | (uintptr_t)router) & 15))
    return -2;
  const size_t lds = (size_t)(2 * n_experts + n_groups) * sizeof(float);
  if (dtype == DT_F32)
    route_rows_sigmoid_kernel<float><<<n_tokens, 256, lds, stream>>>((const float*)x, lda, (const float*)router,
        (const float*)correction, hidden, n_experts, n_groups, keep, top, (int*)chosen, (float*)weights, softmax, group_max,
        (float*)gate);
  else
    route_rows_sigmoid_kernel<bf16_t><<<n_tokens, 256, lds, stream>>>((const bf16_t*)x, lda, (const bf16_t*)router,
        (const float*)correction, hidden, n_experts, n_groups, keep, top, (int*)chosen, (float*)weights, softmax, group_max,
        (float*)gate);
  return LAUNCH_STATUS();
}

// Returns -2 for sizes the fused kernel does not take (the caller then forms the logits with a product of its own).
extern "C" int ta_route_rows_sigmoid(const void* x, int lda, const void* router, const void* correction, int n_tokens,
                                     int hidden, int n_experts, int n_groups, int keep, int top, void* chosen, void* weights,
                                     int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (top <= 0 || top > n_experts || top > WAVE || n_groups < 0) return -1;
  if (n_groups > 0 && (n_experts % n_groups || keep <= 0 || keep > n_groups || keep * (n_experts / n_groups) < top)) return -1;
  const int piece = dtype == DT_F32 ? 4 : 8;
  if (n_experts > RT_MAX_EXPERTS || hidden % piece || lda % piece || hidden > WAVE * RT_ROW_PIECES * piece ||
      (((uintptr_t)x | (uintptr_t)router) & 15))
    return -2;
  const size_t lds = (size_t)(2 * n_experts + n_groups) * sizeof(float);
  if (dtype == DT_F32)
    route_rows_sigmoid_kernel<float><<<n_tokens, 256, lds, stream>>>((const float*)x, lda, (const float*)router,
        (const float*)correction, hidden, n_experts, n_groups, keep, top, (int*)chosen, (float*)weights);
  else
    route_rows_sigmoid_kernel<bf16_t><<<n_tokens, 256, lds, stream>>>((const bf16_t*)x, lda, (const bf16_t*)router,
        (const float*)correction, hidden, n_experts, n_groups, keep, top, (int*)chosen, (float*)weights);
  return LAUNCH_STATUS();
}

extern "C" int ta_expert_act(const void* up, const void* chosen, const void* weights, int n_tokens, int top, int n_experts,
                             int inner, int columns, void* out, int dtype, hipStream_t stream) {
  const size_t total = (size_t)n_tokens * columns;
  if (total == 0) return 0;
  if (columns < n_experts * inner) return -1;
  if (dtype == DT_BF16 && inner % 8 == 0 && columns % 8 == 0 && (((uintptr_t)up | (uintptr_t)out) & 15) == 0) {
    expert_act_vec_kernel<<<rt_blocks(total / 8), 256, 0, stream>>>((const bf16_t*)up, (const int*)chosen,
        (const float*)weights, top, n_experts, inner, columns, (bf16_t*)out, total / 8);
    return LAUNCH_STATUS();
  }
  if (dtype == DT_F32)
    expert_act_kernel<float><<<rt_blocks(total), 256, 0, stream>>>((const float*)up, (const int*)chosen,
        (const float*)weights, top, n_experts, inner, columns, (float*)out, total);
  else
    expert_act_kernel<bf16_t><<<rt_blocks(total), 256, 0, stream>>>((const bf16_t*)up, (const int*)chosen,
        (const float*)weights, top, n_experts, inner, columns, (bf16_t*)out, total);
  return LAUNCH_STATUS();
}

extern "C" int ta_relu2(const void* in, void* out, size_t total, int dtype, hipStream_t stream) {
  if (total == 0) return 0;
  if (dtype == DT_BF16 && total % 8 == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0)
    relu2_vec_kernel<<<rt_blocks(total / 8), 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, total / 8);
  else if (dtype == DT_F32)
    relu2_kernel<float><<<rt_blocks(total), 256, 0, stream>>>((const float*)in, (float*)out, total);
  else
    relu2_kernel<bf16_t><<<rt_blocks(total), 256, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, total);
  return LAUNCH_STATUS();
}
