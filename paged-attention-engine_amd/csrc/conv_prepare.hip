// Short causal convolutions over time on the projected queries, keys and values of an attention
// layer, a weightless RMS norm per query and key head, and the cache write, in one pass.
//
// A projected row holds [q: nh heads of hd | k: nkv heads of hd | v: nkv heads of vd | whatever
// else the product made].  Channel c of the first C = nh hd + nkv (hd + vd) features becomes
//     y_t[c] = sum_j w[c, j] * u_{t - taps + 1 + j}[c]
// over the sequence's own tokens, zeros before its first.  Inputs older than the step's first row
// of the sequence come from the request's state, `conv_tail` [slot][taps - 1][C], oldest first,
// which holds the last taps - 1 projected rows of the sequence in float32 (zeros in a fresh slot);
// `pae_conv_tail_update` moves it on after this kernel has read it.  So a token's result is the
// same however its prompt was cut.  With `norm_heads`, every q and k head is then divided by its
// root mean square over hd (eps inside the root, no weight).  Queries go to `q_out`, keys to
// [block][kv head][offset][hd], values transposed within the page, [block][kv head][vd][offset].
// Sums and norms are float32; a value is rounded to the storage type once, when it is written.
// nkv = 0: the row holds queries only (a layer that reads another layer's keys and values).
#include "common.h"
#include "api.h"

#define CONV_THREADS 128
#define CONV_PER_THREAD 8  // head widths up to CONV_THREADS * CONV_PER_THREAD

// seq_runs[s] = (first flat row, rows in this step, tokens held before the step, unused)
// One workgroup per (token, head): the q heads, then the k heads, then the v heads.
template <typename T>
__global__ __launch_bounds__(CONV_THREADS) void conv_norm_store_kernel(
    const T* __restrict__ proj, int64_t row_stride, T* __restrict__ q_out, int64_t q_stride,
    const int* __restrict__ tok_seq, const int* __restrict__ positions, const int4* __restrict__ seq_runs,
    const int* __restrict__ slots, const float* __restrict__ conv_w, const float* __restrict__ conv_tail,
    int64_t tail_slot_stride, int taps, int nh, int nkv, int hd, int vd, int norm_heads, float eps,
    const int* __restrict__ block_tables, int max_blocks, int bs, T* __restrict__ k_cache, T* __restrict__ v_cache) {
  __shared__ float scratch[CONV_THREADS / PAE_WAVE];
  const int t = blockIdx.x, seg = blockIdx.y;
  const int s = tok_seq[t];
  const int4 run = seq_runs[s];
  const int in_step = t - run.x;  // rows of this sequence before this one in the step
  const int C = nh * hd + nkv * (hd + vd);
  const float* tail = conv_tail ? conv_tail + (int64_t)slots[s] * tail_slot_stride : nullptr;  // [taps - 1][C]
  const bool is_q = seg < nh, is_v = seg >= nh + nkv;
  const int width = is_v ? vd : hd;
  const int c0 = is_v ? (nh + nkv) * hd + (seg - nh - nkv) * vd : seg * hd;
  float mine[CONV_PER_THREAD];
  float ss = 0.f;
#pragma unroll
  for (int n = 0; n < CONV_PER_THREAD; ++n) {
    const int i = threadIdx.x + CONV_THREADS * n;
    mine[n] = 0.f;
    if (i >= width) break;
    const int c = c0 + i;
    float sum = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;  // tap j weighs the input `back` tokens ago
      float x;
      if (back <= in_step) x = to_f32(proj[(int64_t)(t - back) * row_stride + c]);
      else x = tail[(int64_t)(taps - 1 - (back - in_step)) * C + c];
      sum = fmaf(conv_w[(int64_t)c * taps + j], x, sum);
    }
    mine[n] = sum;
    ss = fmaf(sum, sum, ss);
  }
  float inv = 1.f;
  if (norm_heads && !is_v) {
    ss = block_sum<CONV_THREADS / PAE_WAVE>(ss, scratch);
    inv = 1.0f / sqrtf(ss / (float)hd + eps);
  }
  if (is_q) {
    T* dst = q_out + (int64_t)t * q_stride + (int64_t)seg * hd;
#pragma unroll
    for (int n = 0; n < CONV_PER_THREAD; ++n) {
      const int i = threadIdx.x + CONV_THREADS * n;
      if (i >= width) break;
      dst[i] = from_f32<T>(mine[n] * inv);
    }
    return;
  }
  const int pos = positions[t];
  const int off = pos % bs;
  const int64_t block = block_tables[(int64_t)s * max_blocks + pos / bs];
  if (!is_v) {
    T* dst = k_cache + ((block * nkv + (seg - nh)) * bs + off) * hd;
#pragma unroll
    for (int n = 0; n < CONV_PER_THREAD; ++n) {
      const int i = threadIdx.x + CONV_THREADS * n;
      if (i >= width) break;
      dst[i] = from_f32<T>(mine[n] * inv);
    }
  } else {
    T* dst = v_cache + (block * nkv + (seg - nh - nkv)) * (int64_t)vd * bs + off;
#pragma unroll
    for (int n = 0; n < CONV_PER_THREAD; ++n) {
      const int i = threadIdx.x + CONV_THREADS * n;
      if (i >= width) break;
      dst[(int64_t)i * bs] = from_f32<T>(mine[n]);
    }
  }
}

// The state's last taps - 1 inputs moved on by the step's rows: entry j of the new tail is the input
// at (end of step) - keep + j, a row of this step or an entry further on in the old tail (read before
// any entry at or above it is written: j ascends).
template <typename T>
__global__ void conv_tail_update_kernel(const T* __restrict__ proj, int64_t row_stride, const int4* __restrict__ seq_runs,
                                        const int* __restrict__ slots, float* __restrict__ conv_tail,
                                        int64_t tail_slot_stride, int taps, int C) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int4 run = seq_runs[s];
  float* tail = conv_tail + (int64_t)slots[s] * tail_slot_stride;
  const int keep = taps - 1, n = run.y;
  for (int j = 0; j < keep; ++j) {
    const int r = n - keep + j;
    tail[(int64_t)j * C + c] = r >= 0 ? to_f32(proj[(int64_t)(run.x + r) * row_stride + c]) : tail[(int64_t)(j + n) * C + c];
  }
}

extern "C" int pae_conv_norm_store(int dtype, const void* proj, int64_t row_stride, void* q_out, int64_t q_stride,
                                   int num_tokens, int num_seqs, const int* tok_seq, const int* positions,
                                   const int* seq_runs, const int* slots, const float* conv_w, float* conv_tail,
                                   int64_t tail_slot_stride, int taps, int nh, int nkv, int hd, int vd, int norm_heads,
                                   float eps, const int* block_tables, int max_blocks, int bs, void* k_cache,
                                   void* v_cache, hipStream_t stream) {
  PAE_REQUIRE(nh > 0 && nkv >= 0 && hd > 0 && vd > 0, "conv_norm_store: bad head sizes nh=%d nkv=%d hd=%d vd=%d", nh, nkv,
              hd, vd);
  PAE_REQUIRE(hd <= CONV_THREADS * CONV_PER_THREAD && vd <= CONV_THREADS * CONV_PER_THREAD,
              "conv_norm_store: head widths %d / %d exceed %d", hd, vd, CONV_THREADS * CONV_PER_THREAD);
  PAE_REQUIRE(taps >= 1 && taps <= 64, "conv_norm_store: %d taps (1..64)", taps);
  PAE_REQUIRE(taps == 1 || conv_tail, "conv_norm_store: a convolution of %d taps needs the requests' state", taps);
  const int64_t C = (int64_t)nh * hd + (int64_t)nkv * (hd + vd);
  PAE_REQUIRE(row_stride >= C && q_stride >= (int64_t)nh * hd, "conv_norm_store: row strides %lld / %lld too small",
              (long long)row_stride, (long long)q_stride);
  PAE_REQUIRE(tok_seq && positions && seq_runs && slots && conv_w && q_out && proj, "conv_norm_store: missing operands");
  PAE_REQUIRE(nkv == 0 || (bs > 0 && max_blocks > 0 && k_cache && v_cache && block_tables),
              "conv_norm_store: a cache write needs tables and pools");
  PAE_REQUIRE(nh + 2 * nkv <= 65535, "conv_norm_store: %d heads exceed the grid", nh + 2 * nkv);
  if (num_tokens <= 0) return 0;
  dim3 grid(num_tokens, nh + 2 * nkv);
  dim3 tail_grid((unsigned)((C + 255) / 256), num_seqs);
#define CONV_LAUNCH(T)                                                                                                  \
  do {                                                                                                                  \
    conv_norm_store_kernel<T><<<grid, CONV_THREADS, 0, stream>>>(                                                       \
        (const T*)proj, row_stride, (T*)q_out, q_stride, tok_seq, positions, (const int4*)seq_runs, slots, conv_w,      \
        conv_tail, tail_slot_stride, taps, nh, nkv, hd, vd, norm_heads, eps, block_tables, max_blocks, bs, (T*)k_cache, \
        (T*)v_cache);                                                                                                   \
    if (taps > 1)                                                                                                       \
      conv_tail_update_kernel<T><<<tail_grid, 256, 0, stream>>>((const T*)proj, row_stride, (const int4*)seq_runs,      \
                                                                slots, conv_tail, tail_slot_stride, taps, (int)C);      \
  } while (0)
  if (dtype == PAE_F32) CONV_LAUNCH(float);
  else if (dtype == PAE_BF16) CONV_LAUNCH(bf16_t);
  else return pae_fail("conv_norm_store: unknown dtype code %d", dtype);
#undef CONV_LAUNCH
  return pae_check_launch("conv_norm_store");
}
