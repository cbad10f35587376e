// Products of a routed feed-forward over sorted tokens: every tile of BM rows belongs to one expert and is multiplied
// with that expert's matrix alone.  bfloat16 operands, float accumulation on the matrix cores
// (v_mfma_f32_32x32x16_bf16), staged through LDS as in gemm_bf16.hip; and the two small kernels around them: the one
// that sorts a step's (token, chosen expert) pairs into such tiles, and the one that adds a token's experts up.
#include "common.h"

typedef __bf16 gg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gg_floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ void gg_store(float* p, float v) { *p = v; }
__device__ __forceinline__ void gg_store(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }

#define GG_MAX_EXPERTS 256

// chosen: int [n_entries] (entry i = token i / top, its pick i % top; a value outside 0..n_experts-1 is passed over).
// Every expert's entries get consecutive slots, the expert's run starting at a multiple of `bm` slots:
//   slot_of[i] = the entry's slot (or -1), row_of[slot] = the entry's token (or -1 for a slot that only fills a tile up),
//   tile_expert[tile] = the expert of slots tile * bm .. + bm - 1 (or -1 for a tile past the last run).
// row_of has n_tiles * bm entries, tile_expert n_tiles, n_tiles >= n_entries / bm + n_experts.  One workgroup; the
// order of an expert's entries among themselves is whatever order the counter was reached in, which no result depends on.
__global__ void __launch_bounds__(1024)
expert_slots_kernel(const int* __restrict__ chosen, int n_entries, int top, int n_experts, int bm, int n_tiles,
                    int* __restrict__ slot_of, int* __restrict__ row_of, int* __restrict__ tile_expert) {
  __shared__ int count_s[GG_MAX_EXPERTS], start_s[GG_MAX_EXPERTS];
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) count_s[e] = 0;
  for (int s = threadIdx.x; s < n_tiles * bm; s += blockDim.x) row_of[s] = -1;
  for (int t = threadIdx.x; t < n_tiles; t += blockDim.x) tile_expert[t] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < n_entries; i += blockDim.x) {
    const int e = chosen[i];
    slot_of[i] = (e >= 0 && e < n_experts) ? atomicAdd(&count_s[e], 1) : -1;      // for now: the entry's rank in its run
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < n_experts; ++e) {
      start_s[e] = at;
      at += (count_s[e] + bm - 1) / bm * bm;
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x)
    for (int t = start_s[e] / bm; t < (start_s[e] + count_s[e] + bm - 1) / bm; ++t) tile_expert[t] = e;
  for (int i = threadIdx.x; i < n_entries; i += blockDim.x) {
    const int e = chosen[i];
    if (e < 0 || e >= n_experts) continue;
    const int slot = start_s[e] + slot_of[i];
    slot_of[i] = slot;
    row_of[slot] = i / top;
  }
}

// C[slot, :N] = A[row_of[slot], :K] . W_e[:N, :K]^T for every slot of every tile, W_e = W + e * expert_stride elements
// with rows `ldw` apart, e = tile_expert[tile].  row_of null: A's rows are the slots themselves.  A slot that only fills
// a tile up (row_of < 0) is computed from row 0 and never read by anyone.  K, lda, ldw and expert_stride multiples
// of 8, pointers 16-byte aligned.
template <int BM, int BN, int BK, typename OutT, int AHEAD = 3>
__global__ void __launch_bounds__(256)
grouped_gemm_bf16_kernel(const bf16_t* __restrict__ A, int lda, const int* __restrict__ row_of,
                         const int* __restrict__ tile_expert, const bf16_t* __restrict__ W, long expert_stride, int ldw,
                         OutT* __restrict__ C, int ldc, int N, int K) {
  constexpr int WM = BM / 2, WN = BN / 2, TMI = WM / 32, TNI = WN / 32;
  constexpr int GB_LDS = BK + 8, CPR = BK / 8;
  constexpr int A_CHUNKS = BM * CPR / 256, W_CHUNKS = BN * CPR / 256;
  const int expert = scalar_int(tile_expert + blockIdx.y);
  if (expert < 0) return;                                   // a tile past the last run
  __shared__ __attribute__((aligned(16))) uint16_t a_s[2][BM * GB_LDS];
  __shared__ __attribute__((aligned(16))) uint16_t w_s[2][BN * GB_LDS];
  __shared__ int src_s[BM];
  const int tid = threadIdx.x, lane = tid & 63, wave = wave_index();
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  for (int r = tid; r < BM; r += 256) src_s[r] = row_of ? max(row_of[m0 + r], 0) : m0 + r;
  __syncthreads();
  const bf16_t* We = W + (size_t)expert * expert_stride;
  gg_floatx16 acc[TMI][TNI];
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  uint4 a_reg[AHEAD][A_CHUNKS], w_reg[AHEAD][W_CHUNKS];
  int a_row[A_CHUNKS];
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) a_row[i] = src_s[(tid + i * 256) / CPR];
  auto fetch = [&](int k0, uint4 (&a_now)[A_CHUNKS], uint4 (&w_now)[W_CHUNKS]) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int k = min(k0 + (c % CPR) * 8, K - 8);
      a_now[i] = *reinterpret_cast<const uint4*>(A + (size_t)a_row[i] * lda + k);
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int c = tid + i * 256;
      const int n = min(n0 + c / CPR, N - 1), k = min(k0 + (c % CPR) * 8, K - 8);
      w_now[i] = *reinterpret_cast<const uint4*>(We + (size_t)n * ldw + k);
    }
  };
  auto stash = [&](int buf, int k0, const uint4 (&a_now)[A_CHUNKS], const uint4 (&w_now)[W_CHUNKS]) {
    const uint4 zero = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int c = tid + i * 256;
      uint4 v = a_now[i];
      if (k0 + (c % CPR) * 8 >= K) v = zero;
      *reinterpret_cast<uint4*>(a_s[buf] + (c / CPR) * GB_LDS + (c % CPR) * 8) = v;
    }
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int c = tid + i * 256;
      uint4 v = w_now[i];
      if (k0 + (c % CPR) * 8 >= K) v = zero;
      *reinterpret_cast<uint4*>(w_s[buf] + (c / CPR) * GB_LDS + (c % CPR) * 8) = v;
    }
  };
#pragma unroll
  for (int j = 0; j < AHEAD; ++j) fetch(j * BK, a_reg[j], w_reg[j]);
  stash(0, 0, a_reg[0], w_reg[0]);
  __syncthreads();
  int buf = 0;
  for (int k_round = 0; k_round < K; k_round += AHEAD * BK) {
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) {
      const int k0 = k_round + j * BK;
      if (k0 < K) {
        fetch(k0 + AHEAD * BK, a_reg[j], w_reg[j]);
#pragma unroll
        for (int ks = 0; ks < BK; ks += 16) {
          gg_bf16x8 af[TMI], bf[TNI];
#pragma unroll
          for (int i = 0; i < TMI; ++i)
            af[i] = *reinterpret_cast<const gg_bf16x8*>(a_s[buf] + (wm * WM + i * 32 + (lane & 31)) * GB_LDS + ks + 8 * (lane >> 5));
#pragma unroll
          for (int jn = 0; jn < TNI; ++jn)
            bf[jn] = *reinterpret_cast<const gg_bf16x8*>(w_s[buf] + (wn * WN + jn * 32 + (lane & 31)) * GB_LDS + ks + 8 * (lane >> 5));
#pragma unroll
          for (int i = 0; i < TMI; ++i)
#pragma unroll
            for (int jn = 0; jn < TNI; ++jn)
              acc[i][jn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[jn], acc[i][jn], 0, 0, 0);
        }
        if (k0 + BK < K) stash(buf ^ 1, k0 + BK, a_reg[(j + 1) % AHEAD], w_reg[(j + 1) % AHEAD]);
        __syncthreads();
        buf ^= 1;
      }
    }
  }
  // Lane l holds column l%32 and rows 8*(r/4) + 4*(l/32) + r%4 of each 32x32 tile.
#pragma unroll
  for (int i = 0; i < TMI; ++i)
#pragma unroll
    for (int j = 0; j < TNI; ++j) {
      const int n = n0 + wn * WN + j * 32 + (lane & 31);
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * WM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        gg_store(C + (size_t)m * ldc + n, acc[i][j][r]);
      }
    }
}

// out[t, :] = shared[t, :] (if given; times shared_weight[t], float, if that is given) + sum over the token's picks k of weights[t, k] * rows[slot_of[t * top + k], :]
// (a pick without a slot is passed over).  rows float [*, hidden]; shared and out of type T.
template <typename T>
__global__ void expert_combine_kernel(const float* __restrict__ rows, const int* __restrict__ slot_of,
                                      const float* __restrict__ weights, int top, const T* __restrict__ shared,
                                      T* __restrict__ out, int hidden, size_t total,
                                      const float* __restrict__ shared_weight) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / hidden;
    const int h = (int)(idx - t * hidden);
    float sum = shared ? ld(shared + idx) : 0.f;
    if (shared && shared_weight) sum *= shared_weight[t];
    for (int k = 0; k < top; ++k) {
      const int slot = slot_of[t * top + k];
      if (slot >= 0) sum = fmaf(weights[t * top + k], rows[(size_t)slot * hidden + h], sum);
    }
    st(out + idx, sum);
  }
}

extern "C" int ta_expert_slots(const void* chosen, int n_entries, int top, int n_experts, int bm, int n_tiles,
                               void* slot_of, void* row_of, void* tile_expert, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (n_experts <= 0 || n_experts > GG_MAX_EXPERTS || top <= 0 || bm <= 0 || (long)n_tiles * bm < n_entries ||
      n_tiles < (n_entries + bm - 1) / bm + n_experts)
    return -1;
  expert_slots_kernel<<<1, 1024, 0, stream>>>((const int*)chosen, n_entries, top, n_experts, bm, n_tiles, (int*)slot_of,
                                              (int*)row_of, (int*)tile_expert);
  return LAUNCH_STATUS();
}

// bm: 64 or 128 (the tile height the slots were made for).  C has n_tiles * bm rows.
extern "C" int ta_grouped_gemm_bf16(const void* A, int lda, const void* row_of, const void* tile_expert, int n_tiles, int bm,
                                    const void* W, long expert_stride, int ldw, void* C, int ldc, int N, int K,
                                    int out_dtype, hipStream_t stream) {
  if (n_tiles <= 0 || N <= 0) return 0;
  if ((K & 7) || (lda & 7) || (ldw & 7) || (expert_stride & 7) || K < 8 || (((uintptr_t)A | (uintptr_t)W) & 15)) return -1;
#define GO(BMV, BNV, BKV, TT)                                                                                          \
  grouped_gemm_bf16_kernel<BMV, BNV, BKV, TT><<<dim3((N + BNV - 1) / BNV, n_tiles), 256, 0, stream>>>(                 \
      (const bf16_t*)A, lda, (const int*)row_of, (const int*)tile_expert, (const bf16_t*)W, expert_stride, ldw, (TT*)C, ldc, N, K)
  if (bm == 128) { if (out_dtype == DT_F32) GO(128, 128, 32, float); else GO(128, 128, 32, bf16_t); }
  else if (bm == 64) { if (out_dtype == DT_F32) GO(64, 64, 64, float); else GO(64, 64, 64, bf16_t); }
  else return -1;
#undef GO
  return LAUNCH_STATUS();
}

extern "C" int ta_expert_combine(const void* rows, const void* slot_of, const void* weights, int n_tokens, int top,
                                 const void* shared, void* out, int hidden, int dtype, const void* shared_weight,
                                 hipStream_t stream) {
  const size_t total = (size_t)n_tokens * hidden;
  if (total == 0) return 0;
  const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
  if (dtype == DT_F32)
    expert_combine_kernel<float><<<blocks, 256, 0, stream>>>((const float*)rows, (const int*)slot_of, (const float*)weights,
                                                             top, (const float*)shared, (float*)out, hidden, total,
                                                             (const float*)shared_weight);
  else
    expert_combine_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const float*)rows, (const int*)slot_of, (const float*)weights,
                                                              top, (const bf16_t*)shared, (bf16_t*)out, hidden, total,
                                                              (const float*)shared_weight);
  return LAUNCH_STATUS();
}
