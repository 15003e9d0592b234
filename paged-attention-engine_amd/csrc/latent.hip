// Latent attention: what is cached per token is one normed latent vector c (kv_rank wide) and one
// rotated key part shared by all heads (rot_dim wide); keys and values of the heads are products of c.
//
// A projected row holds [q: nh heads of (nope + rd) | down: kv_rank + rd].  This kernel, one
// workgroup per token:
//   * divides the first kv_rank features of `down` by their root mean square (eps inside the root),
//     multiplies by the norm's weight and writes them to the token's place in the latent pages,
//     [block][offset][kv_rank + rd], features 0 .. kv_rank - 1 (and, if the caller keeps them, to the
//     pages of transposed latents, [block][kv_rank][offset]);
//   * rotates the first `rot` of the last rd features of `down` by the token's angles, pairs
//     (2i, 2i + 1) if `interleaved` else (i, i + rot / 2), and writes all rd behind the latent;
//   * rotates the last rd features of every query head likewise and writes them to
//     q_full[t][head][kv_rank .. kv_rank + rd), where the attention kernel expects them behind the
//     head's query folded into latent space (a product that the caller launches).
// The attention over the pages then scores q_full against the cached row as a whole,
//   score = q_folded . c + q_rotated . k_rotated,
// and takes its values from the first kv_rank features of the same row.
// Statistics, weights and the rotation are float32; a value is rounded to the storage type once.
#include "common.h"
#include "api.h"

template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const T* __restrict__ proj, int64_t row_stride, T* __restrict__ q_full, int64_t qf_stride, int nh, int nope, int rd,
    int rot, int interleaved, int rank, const void* __restrict__ norm_w, int w_is_f32, float eps,
    const float* __restrict__ cos_sin, const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_tables, int max_blocks, int bs, T* __restrict__ latent, T* __restrict__ latent_t) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const T* row = proj + (int64_t)t * row_stride;
  const T* down = row + (int64_t)nh * (nope + rd);
  const int pos = positions[t];
  const int64_t block = block_tables[(int64_t)tok_seq[t] * max_blocks + pos / bs];
  T* cached = latent + (block * bs + pos % bs) * (int64_t)(rank + rd);
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += 256) { const float x = to_f32(down[i]); ss = fmaf(x, x, ss); }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += 256) {
    const T c = from_f32<T>(to_f32(down[i]) * inv * load_param(norm_w, w_is_f32, i));
    cached[i] = c;
    // the same latent transposed within the page, [block][rank][offset], for kernels that read values that way
    if (latent_t) latent_t[(block * rank + i) * bs + pos % bs] = c;
  }
  // rotated parts: "head" nh is the shared key part, heads 0 .. nh - 1 the queries'
  const int half = rot / 2;
  for (int idx = threadIdx.x; idx < (nh + 1) * half; idx += 256) {
    const int h = idx / half, i = idx % half;
    const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
    const float c = cos_sin[((int64_t)t * half + i) * 2], s = cos_sin[((int64_t)t * half + i) * 2 + 1];
    const T* src = h < nh ? row + (int64_t)h * (nope + rd) + nope : down + rank;
    T* dst = h < nh ? q_full + (int64_t)t * qf_stride + (int64_t)h * (rank + rd) + rank : cached + rank;
    const float a = to_f32(src[ia]), b = to_f32(src[ib]);
    dst[ia] = from_f32<T>(a * c - b * s);
    dst[ib] = from_f32<T>(b * c + a * s);
  }
  const int rest = rd - rot;  // features behind the rotated ones pass as they are
  for (int idx = threadIdx.x; idx < (nh + 1) * rest; idx += 256) {
    const int h = idx / rest, i = rot + idx % rest;
    const T* src = h < nh ? row + (int64_t)h * (nope + rd) + nope : down + rank;
    T* dst = h < nh ? q_full + (int64_t)t * qf_stride + (int64_t)h * (rank + rd) + rank : cached + rank;
    dst[i] = src[i];
  }
}

extern "C" int pae_latent_prepare(int dtype, const void* proj, int64_t row_stride, void* q_full, int64_t qf_stride,
                                  int num_tokens, int nh, int nope, int rd, int rot, int interleaved, int rank,
                                  const void* norm_w, int w_is_f32, float eps, const float* cos_sin, const int* positions,
                                  const int* tok_seq, const int* block_tables, int max_blocks, int bs, void* latent,
                                  void* latent_t, hipStream_t stream) {
  PAE_REQUIRE(nh > 0 && nope > 0 && rd >= 0 && rank > 0, "latent_prepare: bad sizes nh=%d nope=%d rd=%d rank=%d", nh, nope, rd,
              rank);
  PAE_REQUIRE(rot >= 0 && rot <= rd && rot % 2 == 0, "latent_prepare: %d rotated features of %d", rot, rd);
  PAE_REQUIRE(rot == 0 || cos_sin, "latent_prepare: a rotation needs its table of cosines and sines");
  PAE_REQUIRE(row_stride >= (int64_t)nh * (nope + rd) + rank + rd, "latent_prepare: row stride %lld too small",
              (long long)row_stride);
  PAE_REQUIRE(qf_stride >= (int64_t)nh * (rank + rd), "latent_prepare: query row stride %lld too small", (long long)qf_stride);
  PAE_REQUIRE(bs > 0 && max_blocks > 0 && latent && block_tables && tok_seq && positions && norm_w && q_full,
              "latent_prepare: missing operands");
  if (num_tokens <= 0) return 0;
  if (dtype == PAE_F32)
    latent_prepare_kernel<float><<<num_tokens, 256, 0, stream>>>(
        (const float*)proj, row_stride, (float*)q_full, qf_stride, nh, nope, rd, rot, interleaved, rank, norm_w, w_is_f32, eps,
        cos_sin, positions, tok_seq, block_tables, max_blocks, bs, (float*)latent, (float*)latent_t);
  else if (dtype == PAE_BF16)
    latent_prepare_kernel<bf16_t><<<num_tokens, 256, 0, stream>>>(
        (const bf16_t*)proj, row_stride, (bf16_t*)q_full, qf_stride, nh, nope, rd, rot, interleaved, rank, norm_w, w_is_f32,
        eps, cos_sin, positions, tok_seq, block_tables, max_blocks, bs, (bf16_t*)latent, (bf16_t*)latent_t);
  else
    return pae_fail("latent_prepare: unknown dtype code %d", dtype);
  return pae_check_launch("latent_prepare");
}

// One small product per head for a few rows (single tokens and short portions):
//   out[m][h][n] = sum_k a[m][h][k] * w[h][n][k],   bfloat16 in and out, float32 sums.
// One wavefront per (head, output feature): its lanes share out k (lane, lane + 64, ..), every row's partial sums
// meet by a butterfly, lane 0 writes.  The weights (a few megabytes for all heads) are read once; with at most 64 rows
// the rows stay in cache.  It stands where the plain product's batched entry would take a workgroup of 64 x 64
// outputs for 8 x 128 of them.
#define HEADS_FEW_ROWS 8  // rows a pass keeps sums for
__global__ __launch_bounds__(256) void heads_product_few_kernel(bf16_t* __restrict__ out, int64_t ldc, int64_t head_c,
                                                                const bf16_t* __restrict__ a, int64_t lda, int64_t head_a,
                                                                const bf16_t* __restrict__ w, int M, int N, int K) {
  const int lane = threadIdx.x % PAE_WAVE, wave = threadIdx.x / PAE_WAVE;
  const int n = blockIdx.x * 4 + wave, h = blockIdx.y;
  if (n >= N) return;
  const bf16_t* wr = w + ((int64_t)h * N + n) * K;
  for (int m0 = 0; m0 < M; m0 += HEADS_FEW_ROWS) {
    float sum[HEADS_FEW_ROWS];
#pragma unroll
    for (int r = 0; r < HEADS_FEW_ROWS; ++r) sum[r] = 0.f;
    for (int k = lane; k < K; k += PAE_WAVE) {
      const float wk = to_f32(wr[k]);
#pragma unroll
      for (int r = 0; r < HEADS_FEW_ROWS; ++r)
        if (m0 + r < M) sum[r] = fmaf(to_f32(a[(int64_t)(m0 + r) * lda + h * head_a + k]), wk, sum[r]);
    }
#pragma unroll
    for (int r = 0; r < HEADS_FEW_ROWS; ++r) {
      const float total = wave_sum(sum[r]);
      if (lane == 0 && m0 + r < M) out[(int64_t)(m0 + r) * ldc + h * head_c + n] = __float2bfloat16(total);
    }
  }
}

extern "C" int pae_heads_product_few(void* out, int64_t ldc, int64_t head_c, const void* a, int64_t lda, int64_t head_a,
                                     const void* w, int M, int N, int K, int heads, hipStream_t stream) {
  PAE_REQUIRE(M >= 0 && N > 0 && K > 0 && heads > 0 && heads <= 65535, "heads_product_few: bad sizes M=%d N=%d K=%d heads=%d", M, N,
              K, heads);
  if (M == 0) return 0;
  heads_product_few_kernel<<<dim3((N + 3) / 4, heads), 256, 0, stream>>>((bf16_t*)out, ldc, head_c, (const bf16_t*)a, lda, head_a,
                                                                       (const bf16_t*)w, M, N, K);
  return pae_check_launch("heads_product_few");
}
