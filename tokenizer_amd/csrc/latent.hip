// Attention over a cached latent: what stands between the joined down-projections and the paged attention kernels
// (the two latents' norms, the rotation of the shared key part, the write of the latent into its pages), products
// head by head with a matrix of the head's own (the query taken into the latent's space, the read-out taken out of
// it), and the rotation of the query heads' tails.
#include "common.h"

#define LT_THREADS 256

// rows: [n_tokens, row_stride].  latent_q[t, :] = rows[t, q_offset : q_offset + q_rank] / rms * q_norm.  The kept row
// of a token is [c | turned tail]: c = rows[t, kv_offset : kv_offset + kv_rank] / rms * kv_norm, and the rot
// coordinates behind it in `rows` with coordinate i < rot / 2 and coordinate i + rot / 2 turned by the angle
// position * rates[i] (float).  It goes into key page [n_pages, 1, page_size, kv_rank + rot] at the token's slot and,
// transposed inside a page, into value page [n_pages, 1, kv_rank + rot, page_size].  slots null or a negative slot:
// nothing is stored.  A workgroup a token.
template <typename T>
__global__ void __launch_bounds__(LT_THREADS)
latent_store_kernel(const T* __restrict__ rows, int row_stride, int q_offset, int q_rank, const float* __restrict__ q_norm,
                    int kv_offset, int kv_rank, const float* __restrict__ kv_norm, int rot, const float* __restrict__ rates,
                    float eps, const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ k_pages,
                    T* __restrict__ v_pages, int page_size, T* __restrict__ latent_q) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = rows + (size_t)t * row_stride;
  float sq = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += LT_THREADS) { const float v = ld(row + q_offset + i); sq += v * v; }
  const float inv_q = 1.0f / sqrtf(block_sum(sq, scratch) / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += LT_THREADS)
    st(latent_q + (size_t)t * q_rank + i, ld(row + q_offset + i) * inv_q * q_norm[i]);
  const int slot = slots ? slots[t] : -1;
  if (slot < 0) return;                                       // (the same for every thread of the workgroup)
  sq = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += LT_THREADS) { const float v = ld(row + kv_offset + i); sq += v * v; }
  const float inv_c = 1.0f / sqrtf(block_sum(sq, scratch) / (float)kv_rank + eps);
  const int page = slot / page_size, off = slot % page_size, width = kv_rank + rot;
  T* k_row = k_pages + ((size_t)page * page_size + off) * width;
  T* v_col = v_pages + (size_t)page * width * page_size + off;
  for (int i = threadIdx.x; i < kv_rank; i += LT_THREADS) {
    const float c = ld(row + kv_offset + i) * inv_c * kv_norm[i];
    st(k_row + i, c);
    st(v_col + (size_t)i * page_size, c);
  }
  const int half = rot / 2;
  const float position = (float)positions[t];
  const T* tail = row + kv_offset + kv_rank;
  for (int i = threadIdx.x; i < half; i += LT_THREADS) {
    float s, c;
    sincosf(position * rates[i], &s, &c);
    const float a = ld(tail + i), b = ld(tail + half + i);
    const float lo = a * c - b * s, hi = b * c + a * s;
    st(k_row + kv_rank + i, lo);
    st(k_row + kv_rank + half + i, hi);
    st(v_col + (size_t)(kv_rank + i) * page_size, lo);
    st(v_col + (size_t)(kv_rank + half + i) * page_size, hi);
  }
}

// out[t, h * out_stride + out_offset + i] for i < rot: the rot coordinates of q[t, h * head_width + tail_offset ...]
// with coordinate i < rot / 2 and coordinate i + rot / 2 turned by position * rates[i].
template <typename T>
__global__ void __launch_bounds__(LT_THREADS)
rotate_tails_kernel(const T* __restrict__ q, int q_stride, int heads, int head_width, int tail_offset, int rot,
                    const float* __restrict__ rates, const int* __restrict__ positions, T* __restrict__ out, int out_row,
                    int out_stride, int out_offset) {
  const int t = blockIdx.x, half = rot / 2;
  const float position = (float)positions[t];
  for (int idx = threadIdx.x; idx < heads * half; idx += LT_THREADS) {
    const int i = idx % half, h = idx / half;           // (threads side by side share a head and differ in the rate)
    float s, c;
    sincosf(position * rates[i], &s, &c);
    const T* src = q + (size_t)t * q_stride + (size_t)h * head_width + tail_offset;
    T* dst = out + (size_t)t * out_row + (size_t)h * out_stride + out_offset;
    const float a = ld(src + i), b = ld(src + half + i);
    st(dst + i, a * c - b * s);
    st(dst + half + i, b * c + a * s);
  }
}

// Products head by head: out[t, h * out_stride + out_offset + n] = sum_k x[t, h * x_stride + x_offset + k] * W[h, n, k],
// W [heads, N, K] contiguous.  Float sums in every dtype.  A workgroup owns 64 rows by 64 columns of one head's
// output; tiles of 16 elements of K go through LDS, and a thread keeps 4 by 4 sums.
#define HL_TILE 64
#define HL_K 16
template <typename T>
__global__ void __launch_bounds__(256)
head_linear_kernel(const T* __restrict__ x, int x_row, int x_stride, int x_offset, const T* __restrict__ W,
                   T* __restrict__ out, int out_row, int out_stride, int out_offset, int M, int N, int K) {
  __shared__ float a_s[HL_K][HL_TILE + 4], w_s[HL_K][HL_TILE + 4];
  const int h = blockIdx.z, m0 = blockIdx.y * HL_TILE, n0 = blockIdx.x * HL_TILE, tid = threadIdx.x;
  const T* a = x + (size_t)h * x_stride + x_offset;
  const T* w = W + (size_t)h * N * K;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += HL_K) {
    for (int idx = tid; idx < HL_TILE * HL_K; idx += 256) {
      const int r = idx / HL_K, kk = idx % HL_K;
      const int m = m0 + r, n = n0 + r, k = k0 + kk;
      a_s[kk][r] = (m < M && k < K) ? ld(a + (size_t)m * x_row + k) : 0.f;
      w_s[kk][r] = (n < N && k < K) ? ld(w + (size_t)n * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < HL_K; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { av[i] = a_s[kk][tm + i]; wv[i] = w_s[kk][tn + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + tm + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tn + j;
      if (n < N) st(out + (size_t)m * out_row + (size_t)h * out_stride + out_offset + n, acc[i][j]);
    }
  }
}

// The same on the matrix cores (v_mfma_f32_32x32x16_bf16) for bfloat16 operands whose rows can be read sixteen bytes at
// a time (K, the heads' offsets and the row strides multiples of eight).  A workgroup of four waves owns 64 rows by 64
// columns of a head's output, a wave a 32 by 32 quarter; steps of 32 elements of K go through LDS.
typedef __bf16 lt_bf16x8 __attribute__((ext_vector_type(8)));
typedef float lt_floatx16 __attribute__((ext_vector_type(16)));
#define HM_BK 32
#define HM_LDS (HM_BK + 8)
__global__ void __launch_bounds__(256)
head_linear_mfma_kernel(const bf16_t* __restrict__ x, int x_row, int x_stride, int x_offset, const bf16_t* __restrict__ W,
                        bf16_t* __restrict__ out, int out_row, int out_stride, int out_offset, int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) uint16_t a_s[2][64 * HM_LDS], w_s[2][64 * HM_LDS];
  const int h = blockIdx.z, m0 = blockIdx.y * 64, n0 = blockIdx.x * 64, tid = threadIdx.x, lane = tid & 63;
  const int wave = wave_index(), wm = wave >> 1, wn = wave & 1;
  const bf16_t* a = x + (size_t)h * x_stride + x_offset;
  const bf16_t* w = W + (size_t)h * N * K;
  // A thread brings one piece of sixteen bytes of each tile a step: row tid / 4, piece tid % 4.
  const int r = tid >> 2, piece = (tid & 3) * 8;
  const int am = min(m0 + r, M - 1), wr = min(n0 + r, N - 1);
  lt_floatx16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  auto fetch = [&](int k0, uint4& av, uint4& wv) {
    const int k = min(k0 + piece, K - 8);
    av = *reinterpret_cast<const uint4*>(a + (size_t)am * x_row + k);
    wv = *reinterpret_cast<const uint4*>(w + (size_t)wr * K + k);
  };
  auto stash = [&](int buf, int k0, uint4 av, uint4 wv) {
    if (k0 + piece >= K) av = wv = make_uint4(0, 0, 0, 0);
    *reinterpret_cast<uint4*>(a_s[buf] + r * HM_LDS + piece) = av;
    *reinterpret_cast<uint4*>(w_s[buf] + r * HM_LDS + piece) = wv;
  };
  uint4 av, wv;
  fetch(0, av, wv);
  stash(0, 0, av, wv);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += HM_BK) {
    const bool more = k0 + HM_BK < K;
    if (more) fetch(k0 + HM_BK, av, wv);
#pragma unroll
    for (int ks = 0; ks < HM_BK; ks += 16) {
      const lt_bf16x8 af = *reinterpret_cast<const lt_bf16x8*>(a_s[buf] + (wm * 32 + (lane & 31)) * HM_LDS + ks + 8 * (lane >> 5));
      const lt_bf16x8 bf = *reinterpret_cast<const lt_bf16x8*>(w_s[buf] + (wn * 32 + (lane & 31)) * HM_LDS + ks + 8 * (lane >> 5));
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bf, acc, 0, 0, 0);
    }
    if (more) stash(buf ^ 1, k0 + HM_BK, av, wv);
    __syncthreads();
    buf ^= 1;
  }
  // Lane l holds column l % 32 and rows 8 (i / 4) + 4 (l / 32) + i % 4 of the wave's 32 by 32 tile.
  const int n = n0 + wn * 32 + (lane & 31);
  if (n < N) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = m0 + wm * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
      if (m < M) st(out + (size_t)m * out_row + (size_t)h * out_stride + out_offset + n, acc[i]);
    }
  }
}

// Few rows (single tokens): a wave owns one output column of one head for up to HS_ROWS rows and reads the column's
// row of W once, sixteen bytes a lane a trip, so that the head's matrix streams from memory once whatever the rows.
#define HS_ROWS 8
__global__ void __launch_bounds__(256)
head_linear_skinny_kernel(const bf16_t* __restrict__ x, int x_row, int x_stride, int x_offset, const bf16_t* __restrict__ W,
                          bf16_t* __restrict__ out, int out_row, int out_stride, int out_offset, int M, int N, int K) {
  const int h = blockIdx.z, lane = threadIdx.x & 63, n = blockIdx.x * 4 + (threadIdx.x >> 6), m0 = blockIdx.y * HS_ROWS;
  if (n >= N) return;
  const bf16_t* a = x + (size_t)h * x_stride + x_offset;
  const bf16_t* w = W + ((size_t)h * N + n) * K;
  float acc[HS_ROWS] = {};
  for (int k = lane * 8; k < K; k += 64 * 8) {
    const uint4 raw = *reinterpret_cast<const uint4*>(w + k);
    const uint32_t ww[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < HS_ROWS; ++i) {
      if (m0 + i >= M) break;
      const uint4 xa = *reinterpret_cast<const uint4*>(a + (size_t)(m0 + i) * x_row + k);
      const uint32_t xw[4] = {xa.x, xa.y, xa.z, xa.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[i] = fmaf(__uint_as_float(ww[j] << 16), __uint_as_float(xw[j] << 16), acc[i]);
        acc[i] = fmaf(__uint_as_float(ww[j] & 0xffff0000u), __uint_as_float(xw[j] & 0xffff0000u), acc[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < HS_ROWS; ++i) {
    if (m0 + i >= M) break;
    const float total = wave_sum(acc[i]);
    if (lane == 0) st(out + (size_t)(m0 + i) * out_row + (size_t)h * out_stride + out_offset + n, total);
  }
}

extern "C" int ta_latent_store(const void* rows, int row_stride, int q_offset, int q_rank, const void* q_norm, int kv_offset,
                               int kv_rank, const void* kv_norm, int rot, const void* rates, float eps, const void* positions,
                               const void* slots, void* k_pages, void* v_pages, int page_size, void* latent_q, int n_tokens,
                               int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (q_rank <= 0 || kv_rank <= 0 || rot < 0 || (rot & 1) || (rot > 0 && !rates) || (slots && (!k_pages || !v_pages || page_size <= 0)))
    return -1;
#define LS(TT) latent_store_kernel<TT><<<n_tokens, LT_THREADS, 0, stream>>>((const TT*)rows, row_stride, q_offset, q_rank, \
    (const float*)q_norm, kv_offset, kv_rank, (const float*)kv_norm, rot, (const float*)rates, eps, (const int*)positions, \
    (const int*)slots, (TT*)k_pages, (TT*)v_pages, page_size, (TT*)latent_q)
  if (dtype == DT_F32) LS(float); else LS(bf16_t);
#undef LS
  return LAUNCH_STATUS();
}

extern "C" int ta_rotate_tails(const void* q, int q_stride, int heads, int head_width, int tail_offset, int rot,
                               const void* rates, const void* positions, void* out, int out_row, int out_stride,
                               int out_offset, int n_tokens, int dtype, hipStream_t stream) {
  if (n_tokens <= 0 || rot == 0) return 0;
  if (rot < 0 || (rot & 1) || heads <= 0 || tail_offset + rot > head_width) return -1;
#define RT(TT) rotate_tails_kernel<TT><<<n_tokens, LT_THREADS, 0, stream>>>((const TT*)q, q_stride, heads, head_width, \
    tail_offset, rot, (const float*)rates, (const int*)positions, (TT*)out, out_row, out_stride, out_offset)
  if (dtype == DT_F32) RT(float); else RT(bf16_t);
#undef RT
  return LAUNCH_STATUS();
}

extern "C" int ta_head_linear(const void* x, int x_row, int x_stride, int x_offset, const void* W, void* out, int out_row,
                              int out_stride, int out_offset, int M, int N, int K, int heads, int dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0 || heads <= 0) return 0;
  if (K <= 0 || heads > 65535) return -1;
  if (dtype == DT_BF16 && K % 8 == 0 && x_row % 8 == 0 && x_stride % 8 == 0 && x_offset % 8 == 0 &&
      (((uintptr_t)x | (uintptr_t)W) & 15) == 0) {
    if (M <= 2 * HS_ROWS) {
      dim3 grid((N + 3) / 4, (M + HS_ROWS - 1) / HS_ROWS, heads);
      head_linear_skinny_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_stride, x_offset, (const bf16_t*)W,
                                                          (bf16_t*)out, out_row, out_stride, out_offset, M, N, K);
      return LAUNCH_STATUS();
    }
    dim3 grid((N + 63) / 64, (M + 63) / 64, heads);
    if (grid.y > 65535) return -1;
    head_linear_mfma_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)x, x_row, x_stride, x_offset, (const bf16_t*)W,
                                                      (bf16_t*)out, out_row, out_stride, out_offset, M, N, K);
    return LAUNCH_STATUS();
  }
  dim3 grid((N + HL_TILE - 1) / HL_TILE, (M + HL_TILE - 1) / HL_TILE, heads);
  if (grid.y > 65535) return -1;
#define HL(TT) head_linear_kernel<TT><<<grid, 256, 0, stream>>>((const TT*)x, x_row, x_stride, x_offset, (const TT*)W, \
    (TT*)out, out_row, out_stride, out_offset, M, N, K)
  if (dtype == DT_F32) HL(float); else HL(bf16_t);
#undef HL
  return LAUNCH_STATUS();
}
