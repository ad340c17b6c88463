// Latent attention: keys and values of all heads are products of one cached latent vector per position.
//
// What a position keeps is the row [c | kr]: the normed latent c (`rank` wide) and one rotated key part kr
// (`rot` wide) that all heads share.  With q_h = [qn_h | qr_h] a head's score is
//   qn_h . (Wuk_h c) + qr_h . kr  =  (Wuk_h^T qn_h) . c + qr_h . kr,
// so attention runs as one key head of width rank + rot that all query heads share, over the paged cache, with
// the query [Wuk_h^T qn_h | rot(qr_h)]; the weighted sum of the cached rows' first `rank` columns then goes
// through Wuv_h.  The cache holds the row twice, as keys [page, 1, slot, rank + rot] and transposed as values
// [page, 1, rank + rot, slot], which is the layout the paged attention kernels read.
#include "common.h"
#include "group_tile.h"

// ---------------------------------------------------------------------------------------------
// One workgroup per token: c = rms_norm(x[:rank]) * weight, kr = rotate(x[rank:]) (pairs (i, i + rot_dims / 2) of
// the first `rot_dims` dims, angle float(pos) * inv_freq[i]); the row goes to the token's page and slot.
// x: 32-bit [T, ldx].  A token whose page id is negative writes nothing.
template <typename TC>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(
    const float* __restrict__ x, long long ldx, const float* __restrict__ weight, float eps, int rank, int rot,
    int rot_dims, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    const int* __restrict__ entry_of, const int* __restrict__ table, int table_width, int block_size,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* src = x + (long long)t * ldx;
  float ss = 0.f;
  for (int c = threadIdx.x; c < rank; c += blockDim.x) ss += src[c] * src[c];
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  const int pos = positions[t];
  const int page = table[(long long)entry_of[t] * table_width + pos / block_size];
  if (page < 0) return;
  const int slot = pos % block_size;
  const int width = rank + rot, half = rot_dims / 2;
  TC* krow = k_cache + ((long long)page * block_size + slot) * width;
  TC* vcol = v_cache + (long long)page * width * block_size + slot;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float value;
    if (c < rank) {
      value = src[c] * inv * weight[c];
    } else {
      const int i = c - rank;
      if (i < rot_dims) {
        const int pair = i < half ? i : i - half;
        float sn, cs;
        sincosf((float)pos * inv_freq[pair], &sn, &cs);
        const float lo = src[rank + pair], hi = src[rank + pair + half];
        value = i < half ? lo * cs - hi * sn : hi * cs + lo * sn;
      } else {
        value = src[c];
      }
    }
    const TC stored = from_float<TC>(value);
    krow[c] = stored;
    vcol[(long long)c * block_size] = stored;
  }
}

// The rotated part of every query head: out[t, h, out_offset + i] = rotate(q[t, h, q_offset + i]), i < rot.
// q: [T, ldq] with `q_head` columns per head; out: [T, heads, out_head].  One thread per (token, head, pair or
// unrotated dim).
template <typename T>
__global__ void latent_q_rotate_kernel(const T* __restrict__ q, long long ldq, int q_head, int q_offset,
                                       T* __restrict__ out, int out_head, int out_offset, int heads, int rot,
                                       int rot_dims, const int* __restrict__ positions,
                                       const float* __restrict__ inv_freq, long long total) {
  const int half = rot_dims / 2;
  const int per_head = rot - half;       // `half` pairs, then the dims that pass unchanged
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int i = (int)(idx % per_head);
  const long long th = idx / per_head;
  const int h = (int)(th % heads), t = (int)(th / heads);
  const T* src = q + (long long)t * ldq + (long long)h * q_head + q_offset;
  T* dst = out + ((long long)t * heads + h) * out_head + out_offset;
  if (i < half) {
    float sn, cs;
    sincosf((float)positions[t] * inv_freq[i], &sn, &cs);
    const float lo = to_float<T>(src[i]), hi = to_float<T>(src[i + half]);
    dst[i] = from_float<T>(lo * cs - hi * sn);
    dst[i + half] = from_float<T>(hi * cs + lo * sn);
  } else {
    dst[i + half] = src[i + half];
  }
}

// ---------------------------------------------------------------------------------------------
// A product per head: out[t, h, n] = sum_k a[t, h, k] * w[h, n, k].  a: row stride lda, head stride sa; out: row
// stride ldo, head stride so; w contiguous [heads, N, K].  Grid (ceil(T / 64), ceil(N / 64), heads), 256 threads,
// each 4 x 4 outputs; K in steps of 16 through LDS; an output element is one FMA chain in k order, so it does not
// depend on the other rows of the launch.
template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void head_linear_kernel(const TA* __restrict__ a, long long lda, long long sa,
                                                          const TW* __restrict__ w, TO* __restrict__ out,
                                                          long long ldo, long long so, int M, int N, int K) {
  __shared__ float As[16][64 + 4];
  __shared__ float Ws[16][64 + 4];
  const int h = blockIdx.z;
  const int m0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
  const TA* ah = a + (long long)h * sa;
  const TW* wh = w + (long long)h * N * K;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int i = threadIdx.x; i < 64 * 16; i += 256) {
      const int r = i >> 4, kk = i & 15;
      const int m = m0 + r, n = n0 + r, k = k0 + kk;
      As[kk][r] = (m < M && k < K) ? to_float<TA>(ah[(long long)m * lda + k]) : 0.f;
      Ws[kk][r] = (n < N && k < K) ? to_float<TW>(wh[(long long)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[(long long)m * ldo + (long long)h * so + n] = from_float<TO>(acc[i][j]);
    }
  }
}

// The same product on the matrix cores (bfloat16 in and out; K a multiple of 8, 16-byte rows): tiles of 128 tokens
// x 128 outputs of one head, see group_tile.h.  Grid (ceil(T / 128), ceil(N / 128), heads).
__global__ __launch_bounds__(256) void head_linear_mma_kernel(const __bf16* __restrict__ a, long long lda, long long sa,
                                                              const __bf16* __restrict__ w, __bf16* __restrict__ out,
                                                              long long ldo, long long so, int M, int N, int K) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int h = blockIdx.z, m0 = blockIdx.x * GT_TILE, n0 = blockIdx.y * GT_TILE;
  const __bf16* ah = a + (long long)h * sa;
  const __bf16* wh = w + (long long)h * N * K;
  gt_f32x4 acc[4][4];
  group_tile_mma([&](int r) -> const __bf16* { return m0 + r < M ? ah + (long long)(m0 + r) * lda : nullptr; },
                 [&](int r) -> const __bf16* { return n0 + r < N ? wh + (long long)(n0 + r) * K : nullptr; }, K, lds, acc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 15, lg = lane >> 4;
#pragma unroll
  for (int tm = 0; tm < 4; ++tm) {
    const int m = m0 + wm * 64 + tm * 16 + lr;
    if (m >= M) continue;
    __bf16* dst = out + (long long)m * ldo + (long long)h * so;
#pragma unroll
    for (int tn = 0; tn < 4; ++tn)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + wn * 64 + tn * 16 + lg * 4 + i;
        if (n < N) dst[n] = (__bf16)acc[tn][tm][i];
      }
  }
}

// ---------------------------------------------------------------------------------------------
extern "C" int vk_latent_kv_write(const float* x, long long ldx, const float* weight, float eps, int rank, int rot,
                                  int rot_dims, const int* positions, const float* inv_freq, const int* entry_of,
                                  const int* table, int table_width, int block_size, void* k_cache, void* v_cache,
                                  int cache_dtype, int num_tokens, void* stream) {
  if (num_tokens <= 0) return 0;
  if (rank < 1 || rot < 0 || rot_dims < 0 || rot_dims > rot || (rot_dims & 1) || block_size < 1 || table_width < 1)
    return VK_BAD_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (cache_dtype == DT_F32)
    latent_kv_write_kernel<float><<<num_tokens, 256, 0, s>>>(x, ldx, weight, eps, rank, rot, rot_dims, positions,
                                                             inv_freq, entry_of, table, table_width, block_size,
                                                             (float*)k_cache, (float*)v_cache);
  else if (cache_dtype == DT_BF16)
    latent_kv_write_kernel<bf16_t><<<num_tokens, 256, 0, s>>>(x, ldx, weight, eps, rank, rot, rot_dims, positions,
                                                              inv_freq, entry_of, table, table_width, block_size,
                                                              (bf16_t*)k_cache, (bf16_t*)v_cache);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_latent_q_rotate(const void* q, long long ldq, int q_head, int q_offset, void* out, int out_head,
                                  int out_offset, int heads, int rot, int rot_dims, const int* positions,
                                  const float* inv_freq, int dtype, int num_tokens, void* stream) {
  if (num_tokens <= 0 || rot <= 0) return 0;
  if (heads < 1 || rot_dims < 0 || rot_dims > rot || (rot_dims & 1)) return VK_BAD_ARGUMENT;
  const long long total = (long long)num_tokens * heads * (rot - rot_dims / 2);
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32)
    latent_q_rotate_kernel<float><<<blocks, 256, 0, s>>>((const float*)q, ldq, q_head, q_offset, (float*)out, out_head,
                                                         out_offset, heads, rot, rot_dims, positions, inv_freq, total);
  else if (dtype == DT_BF16)
    latent_q_rotate_kernel<bf16_t><<<blocks, 256, 0, s>>>((const bf16_t*)q, ldq, q_head, q_offset, (bf16_t*)out,
                                                          out_head, out_offset, heads, rot, rot_dims, positions,
                                                          inv_freq, total);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_head_linear(const void* a, int a_dtype, long long lda, long long sa, const void* w, int w_dtype,
                              void* out, int out_dtype, long long ldo, long long so, int M, int N, int K, int heads,
                              void* stream) {
  if (M <= 0 || N <= 0 || heads <= 0) return 0;
  if (K < 1 || heads > 65535) return VK_BAD_ARGUMENT;
  dim3 grid((M + 63) / 64, (N + 63) / 64, heads);
  if (grid.y > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  if (a_dtype == DT_F32 && w_dtype == DT_F32 && out_dtype == DT_F32)
    head_linear_kernel<float, float, float><<<grid, 256, 0, s>>>((const float*)a, lda, sa, (const float*)w, (float*)out,
                                                                 ldo, so, M, N, K);
  else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_BF16 && K % 8 == 0 && lda % 8 == 0 && sa % 8 == 0 &&
           (((uintptr_t)a | (uintptr_t)w) & 15) == 0) {
    static bool sized = false;
    if (!sized) {
      hipError_t e = hipFuncSetAttribute((const void*)head_linear_mma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         GT_LDS_BYTES);
      if (e != hipSuccess) return (int)e;
      sized = true;
    }
    dim3 wide((M + GT_TILE - 1) / GT_TILE, (N + GT_TILE - 1) / GT_TILE, heads);
    head_linear_mma_kernel<<<wide, 256, GT_LDS_BYTES, s>>>((const __bf16*)a, lda, sa, (const __bf16*)w, (__bf16*)out, ldo,
                                                           so, M, N, K);
  } else if (a_dtype == DT_BF16 && w_dtype == DT_BF16 && out_dtype == DT_BF16)
    head_linear_kernel<bf16_t, bf16_t, bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)a, lda, sa, (const bf16_t*)w,
                                                                    (bf16_t*)out, ldo, so, M, N, K);
  else if (a_dtype == DT_BF16 && w_dtype == DT_F32 && out_dtype == DT_BF16)
    head_linear_kernel<bf16_t, float, bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)a, lda, sa, (const float*)w,
                                                                   (bf16_t*)out, ldo, so, M, N, K);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}
