// Causal attention over the paged cache, one wavefront per (token, query head).
//
// This is the kernel every size goes through in float32 and the one bfloat16
// falls back to when the matrix-core kernels do not take a shape.  A step's
// tokens are flat: token t belongs to sequence tok_seq[t] and stands at
// positions[t]; its keys are the cache slots of positions start..pos of that
// sequence, start = max(0, pos - window + 1) (window 0: every earlier key).  The
// rule is the reference's mask (engine/attention.py:474-487: key j is visible iff
// j <= query position and j < kv length) plus the window, which it lacks.
// KV head j serves query heads j*g .. (j+1)*g-1 (engine/attention.py:72-74).
//
// Keys are walked in chunks of 64 aligned to multiples of 64 from position 0,
// lane = key within the chunk, with an online softmax in float32.  What a
// (token, head) computes therefore depends on nothing but its own position:
// not on how the step was cut, nor on what else is in the batch.
//
// Three things beyond the reference's attention, each switched by a parameter: values of their own
// width `vd` (keys and queries stay `hd` wide), a cap on the scores (s <- cap * tanh(s / cap),
// cap 0: none), and one learned sink per query head, a number that joins the softmax's denominator
// as exp(sink) without a key or a value of its own (sinks null: none).
//
// And four more, for designs that have them: a mask in chunks (`chunked`: the `window` is then a
// chunk length, and position p sees the keys from p - p % window on, chunk borders at multiples of the length from the first token
// of the sequence); a bias by distance, score -= slopes[head] * (p - key) (slopes null: none); a gate
// on the output, out *= sigmoid(gate[token][head][feature]) (gate null: none); and values that are
// the first `vd` features of the key rows themselves (`shared_kv`, one latent row per token that
// serves as key and as value: v_cache is then not read).
#include "common.h"
#include "api.h"

template <typename T, int MAXD>  // MAXD: output features per lane, value width <= 64 * MAXD
__global__ void paged_attention_generic_kernel(
    T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, const int* __restrict__ positions,
    const int* __restrict__ tok_seq, const int* __restrict__ block_tables, int max_blocks, int bs,
    int nh, int nkv, int hd, int vd, float scale, int window, float cap, const float* __restrict__ sinks,
    int chunked, const float* __restrict__ slopes, const T* __restrict__ gate, int64_t gate_stride, int shared_kv) {
  extern __shared__ float lds[];  // [hd] query, [64] probabilities
  float* q_lds = lds;
  float* p_lds = lds + hd;
  const int t = blockIdx.x;
  const int head = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = head / (nh / nkv);
  const int pos = positions[t];
  const int* table = block_tables + (int64_t)tok_seq[t] * max_blocks;
  const int start = window <= 0 ? 0 : (chunked ? pos - pos % window : (pos - window + 1 > 0 ? pos - window + 1 : 0));
  const float slope = slopes ? slopes[head] : 0.f;

  const T* q_row = q + (int64_t)t * q_stride + (int64_t)head * hd;
  for (int d = lane; d < hd; d += PAE_WAVE) q_lds[d] = to_f32(q_row[d]);
  __syncthreads();

  float acc[MAXD];
#pragma unroll
  for (int i = 0; i < MAXD; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int base = (start / PAE_WAVE) * PAE_WAVE; base <= pos; base += PAE_WAVE) {
    const int key = base + lane;
    const bool valid = key >= start && key <= pos;
    int row = 0;  // this lane's key row in the pool, in units of head_dim elements
    float s = -INFINITY;
    if (valid) {
      const int blk = table[key / bs];
      row = (blk * nkv + kvh) * bs + key % bs;
      const T* kr = k_cache + (int64_t)row * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(q_lds[d], to_f32(kr[d]), dot);
      s = dot * scale;
      if (slopes) s -= slope * (float)(pos - key);
      if (cap > 0.f) s = cap * tanhf(s / cap);
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: every chunk holds a valid key
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);        // 0 on the first chunk (m = -inf)
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_lds[lane] = p;
    __syncthreads();
    const int first = (start > base ? start - base : 0);
    const int last = (pos - base < PAE_WAVE - 1 ? pos - base : PAE_WAVE - 1);
#pragma unroll
    for (int i = 0; i < MAXD; ++i) acc[i] *= alpha;
    for (int j = first; j <= last; ++j) {
      const float pj = p_lds[j];
      const int rj = __shfl(row, j, PAE_WAVE);
      // values are transposed within a page: [block][kv head][feature][offset in page]; shared with
      // the keys they are the head of the key row
      const T* vr = shared_kv ? k_cache + (int64_t)rj * hd : v_cache + (int64_t)(rj / bs) * bs * vd + rj % bs;
      const int64_t step = shared_kv ? 1 : bs;
#pragma unroll
      for (int i = 0; i < MAXD; ++i) {
        const int d = lane + i * PAE_WAVE;
        if (d < vd) acc[i] = fmaf(pj, to_f32(vr[(int64_t)d * step]), acc[i]);
      }
    }
    __syncthreads();
  }
  T* o = out + (int64_t)t * out_stride + (int64_t)head * vd;
  float keep = 1.f;  // what the sums keep when the sink raises the reference point
  if (sinks) {
    const float sink = sinks[head];
    const float m_all = fmaxf(m, sink);
    keep = expf(m - m_all);
    l = l * keep + expf(sink - m_all);
  }
  const float inv = keep / l;
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = lane + i * PAE_WAVE;
    if (d < vd) {
      float v = acc[i] * inv;
      if (gate) v *= 1.0f / (1.0f + expf(-to_f32(gate[(int64_t)t * gate_stride + (int64_t)head * vd + d])));
      o[d] = from_f32<T>(v);
    }
  }
}

template <typename T>
static int launch_generic(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                          const void* v_cache, const int* positions, const int* tok_seq,
                          const int* block_tables, int max_blocks, int bs, int num_tokens, int nh, int nkv,
                          int hd, int vd, float scale, int window, float cap, const float* sinks, int chunked,
                          const float* slopes, const void* gate, int64_t gate_stride, int shared_kv,
                          hipStream_t stream) {
  dim3 grid(num_tokens, nh);
  const size_t lds = (size_t)(hd + PAE_WAVE) * sizeof(float);
#define PAE_LAUNCH(MAXD)                                                                              \
  paged_attention_generic_kernel<T, MAXD><<<grid, PAE_WAVE, lds, stream>>>(                           \
      (T*)out, out_stride, (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, positions,    \
      tok_seq, block_tables, max_blocks, bs, nh, nkv, hd, vd, scale, window, cap, sinks, chunked,   \
      slopes, (const T*)gate, gate_stride, shared_kv)
  if (vd <= 64) PAE_LAUNCH(1);
  else if (vd <= 128) PAE_LAUNCH(2);
  else if (vd <= 192) PAE_LAUNCH(3);
  else if (vd <= 256) PAE_LAUNCH(4);
  else PAE_LAUNCH(8);
#undef PAE_LAUNCH
  return pae_check_launch("paged_attention_generic");
}

extern "C" int pae_paged_attention_masked(int dtype, void* out, int64_t out_stride, const void* q,
                                          int64_t q_stride, const void* k_cache, const void* v_cache,
                                          const int* positions, const int* tok_seq,
                                          const int* block_tables, int max_blocks, int bs,
                                          int num_tokens, int nh, int nkv, int hd, int vd, float scale,
                                          int window, float cap, const float* sinks, int chunked,
                                          const float* slopes, const void* gate, int64_t gate_stride, int shared_kv,
                                          hipStream_t stream) {
  PAE_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "attention: %d query heads over %d key/value heads", nh, nkv);
  PAE_REQUIRE(hd > 0 && hd <= 1024, "attention: head_dim %d is outside 1..1024", hd);
  PAE_REQUIRE(vd > 0 && vd <= 512, "attention: value width %d is outside 1..512", vd);
  PAE_REQUIRE(!shared_kv || (nkv == 1 && vd <= hd), "attention: values shared with the keys need one key head at least as wide");
  PAE_REQUIRE(!gate || gate_stride >= (int64_t)nh * vd, "attention: gate row stride %lld too small", (long long)gate_stride);
  PAE_REQUIRE(shared_kv || v_cache, "attention: no values");
  PAE_REQUIRE(bs > 0 && max_blocks > 0, "attention: bad cache geometry bs=%d max_blocks=%d", bs, max_blocks);
  PAE_REQUIRE(window >= 0, "attention: negative window %d", window);
  PAE_REQUIRE(cap >= 0.f, "attention: negative score cap %g", (double)cap);
  PAE_REQUIRE(nh <= 65535, "attention: %d query heads exceed the grid", nh);
  if (num_tokens <= 0) return 0;
  if (dtype == PAE_F32)
    return launch_generic<float>(out, out_stride, q, q_stride, k_cache, v_cache, positions, tok_seq, block_tables,
                                 max_blocks, bs, num_tokens, nh, nkv, hd, vd, scale, window, cap, sinks, chunked, slopes, gate,
                                 gate_stride, shared_kv, stream);
  if (dtype == PAE_BF16)
    return launch_generic<bf16_t>(out, out_stride, q, q_stride, k_cache, v_cache, positions, tok_seq, block_tables,
                                  max_blocks, bs, num_tokens, nh, nkv, hd, vd, scale, window, cap, sinks, chunked, slopes, gate,
                                  gate_stride, shared_kv, stream);
  return pae_fail("attention: unknown dtype code %d", dtype);
}

extern "C" int pae_paged_attention_capped(int dtype, void* out, int64_t out_stride, const void* q,
                                          int64_t q_stride, const void* k_cache, const void* v_cache,
                                          const int* positions, const int* tok_seq,
                                          const int* block_tables, int max_blocks, int bs,
                                          int num_tokens, int nh, int nkv, int hd, int vd, float scale,
                                          int window, float cap, const float* sinks, hipStream_t stream) {
  PAE_REQUIRE(vd > 0 && vd <= 256, "attention: value width %d is outside 1..256", vd);
  return pae_paged_attention_masked(dtype, out, out_stride, q, q_stride, k_cache, v_cache, positions, tok_seq,
                                    block_tables, max_blocks, bs, num_tokens, nh, nkv, hd, vd, scale, window, cap, sinks,
                                    0, nullptr, nullptr, 0, 0, stream);
}

extern "C" int pae_paged_attention_generic(int dtype, void* out, int64_t out_stride, const void* q,
                                           int64_t q_stride, const void* k_cache, const void* v_cache,
                                           const int* positions, const int* tok_seq,
                                           const int* block_tables, int max_blocks, int bs,
                                           int num_tokens, int nh, int nkv, int hd, float scale,
                                           int window, hipStream_t stream) {
  PAE_REQUIRE(hd > 0 && hd <= 256, "attention: head_dim %d is outside 1..256", hd);
  return pae_paged_attention_capped(dtype, out, out_stride, q, q_stride, k_cache, v_cache, positions, tok_seq,
                                    block_tables, max_blocks, bs, num_tokens, nh, nkv, hd, hd, scale, window, 0.f,
                                    nullptr, stream);
}
