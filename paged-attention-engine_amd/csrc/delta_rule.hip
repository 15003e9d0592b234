// The gated delta rule: a recurrent mixer whose per-request state is one matrix per head and the
// last few inputs of its short convolutions.
//
// A step's projected rows hold, per token,
//   [q: G heads of D | k: G heads of D | v: H heads of V | gate: H heads of V | b: H | a: H]
// (G key heads serve H value heads, head h reads key head h / (H / G)).  Four kernels:
//
//   delta_prepare      the first C = 2 G D + H V columns pass a causal convolution over time, one
//                      filter of `taps` taps per column (the last tap is the current token's; what
//                      came before the step is read from the request's state, zeros at its start),
//                      and SiLU; q and k heads become unit vectors, x / sqrt(sum x^2 + unit_eps), q
//                      also times D^-1/2; beta = sigmoid(b); decay = exp(-exp(A_log) softplus(a + dt)).
//   delta_conv_tail    the state's last taps - 1 inputs are moved on by the step's rows.
//   delta_recurrence   per head and token, in this order:  S <- decay S;  u = beta (v - S^T k);
//                      S <- S + k u^T;  o = S^T q.  Columns of S are independent of each other, so a
//                      column is owned by a group of lanes that hold it in registers from the step's
//                      first token to its last; the lanes of a group share out the D rows.
//   delta_gated_norm   o / sqrt(mean_V(o^2) + eps) * w * silu(gate), rounded to the activation type.
//
// Everything but the projected rows is float32: the convolution's sums, the unit vectors, beta,
// the decay and its logarithm, the state, the read-out and the norm.  The order in which a
// column's sums are formed depends on D alone, so a token's result does not depend on how a
// prompt was cut into steps or on what else the step holds.
#include "common.h"
#include "api.h"

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// seq_runs[s] = (first flat row, rows in this step, tokens held before the step, unused)
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(
    const T* __restrict__ proj, int64_t row_stride, const int* __restrict__ tok_seq, const int* __restrict__ positions,
    const int4* __restrict__ seq_runs, const int* __restrict__ slots, const float* __restrict__ conv_w,
    const float* __restrict__ conv_tail, int64_t tail_slot_stride, int taps, int G, int H, int D, int V,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, float unit_eps, float* __restrict__ q_out,
    float* __restrict__ k_out, float* __restrict__ v_out, float* __restrict__ beta_out, float* __restrict__ decay_out) {
  extern __shared__ float chan[];  // [C] the token's convolved, activated channels
  const int t = blockIdx.x;
  const int s = tok_seq[t];
  const int4 run = seq_runs[s];
  const int in_step = t - run.x;  // rows of this sequence before this one in the step
  const int C = 2 * G * D + H * V;
  const float* tail = conv_tail + (int64_t)slots[s] * tail_slot_stride;  // [taps - 1][C], oldest first
  for (int c = threadIdx.x; c < C; c += 256) {
    float sum = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;  // tap j weighs the input `back` tokens ago
      float x;
      if (back <= in_step) x = to_f32(proj[(int64_t)(t - back) * row_stride + c]);
      else x = tail[(int64_t)(taps - 1 - (back - in_step)) * C + c];
      sum = fmaf(conv_w[(int64_t)c * taps + j], x, sum);
    }
    chan[c] = silu_f(sum);
  }
  __syncthreads();
  const int wave = threadIdx.x / PAE_WAVE, lane = threadIdx.x % PAE_WAVE;
  const float q_scale = 1.0f / sqrtf((float)D);
  for (int head = wave; head < 2 * G; head += 4) {  // q heads, then k heads
    const float* x = chan + head * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += PAE_WAVE) ss = fmaf(x[d], x[d], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss + unit_eps);
    const bool is_q = head < G;
    float* dst = is_q ? q_out + ((int64_t)t * G + head) * D : k_out + ((int64_t)t * G + head - G) * D;
    for (int d = lane; d < D; d += PAE_WAVE) dst[d] = is_q ? x[d] * inv * q_scale : x[d] * inv;
  }
  for (int i = threadIdx.x; i < H * V; i += 256) v_out[(int64_t)t * H * V + i] = chan[2 * G * D + i];
  const T* row = proj + (int64_t)t * row_stride;
  for (int h = threadIdx.x; h < H; h += 256) {
    const float b = to_f32(row[C + H * V + h]), a = to_f32(row[C + H * V + H + h]);
    beta_out[(int64_t)t * H + h] = 1.0f / (1.0f + expf(-b));
    decay_out[(int64_t)t * H + h] = expf(-expf(a_log[h]) * softplus_f(a + dt_bias[h]));
  }
}

template <typename T>
__global__ void delta_conv_tail_kernel(const T* __restrict__ proj, int64_t row_stride, const int4* __restrict__ seq_runs,
                                       const int* __restrict__ slots, float* __restrict__ conv_tail,
                                       int64_t tail_slot_stride, int taps, int C) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int4 run = seq_runs[s];
  float* tail = conv_tail + (int64_t)slots[s] * tail_slot_stride;
  const int keep = taps - 1, n = run.y;
  // entry j of the new tail is the input at (end of step) - keep + j: a row of this step, or an entry
  // further on in the old tail (read before any entry at or above it is written: j ascends)
  for (int j = 0; j < keep; ++j) {
    const int r = n - keep + j;  // row of the step, negative: before it
    tail[(int64_t)j * C + c] = r >= 0 ? to_f32(proj[(int64_t)(run.x + r) * row_stride + c]) : tail[(int64_t)(j + n) * C + c];
  }
}

// One group of L lanes per column of S; a lane holds R consecutive rows of its column.
template <int R>
__global__ __launch_bounds__(256) void delta_recurrence_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, const float* __restrict__ beta,
    const float* __restrict__ decay, const int4* __restrict__ seq_runs, const int* __restrict__ slots,
    float* __restrict__ state, int64_t state_slot_stride, int G, int H, int D, int V, int L, float* __restrict__ out) {
  const int s = blockIdx.z, h = blockIdx.y;
  const int col = blockIdx.x * (256 / L) + threadIdx.x / L;
  const int sub = threadIdx.x % L;
  const int4 run = seq_runs[s];
  if (col >= V) return;  // whole groups leave together: the shuffles below stay within a group
  const int g = h / (H / G);
  float* column = state + (int64_t)slots[s] * state_slot_stride + ((int64_t)h * V + col) * D;  // [H][V][D]
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = sub * R + r;
    S[r] = d < D ? column[d] : 0.f;
  }
  for (int i = 0; i < run.y; ++i) {
    const int64_t t = run.x + i;
    const float* kt = k + (t * G + g) * D;
    const float* qt = q + (t * G + g) * D;
    float kr[R], qr[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = sub * R + r;
      kr[r] = d < D ? kt[d] : 0.f;
      qr[r] = d < D ? qt[d] : 0.f;
    }
    const float dec = decay[t * H + h], b = beta[t * H + h], vt = v[(t * H + h) * V + col];
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] = dec * S[r];
      dot = fmaf(S[r], kr[r], dot);
    }
    for (int off = L / 2; off > 0; off >>= 1) dot += __shfl_xor(dot, off, L);
    const float u = b * (vt - dot);
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      S[r] = fmaf(kr[r], u, S[r]);
      o = fmaf(S[r], qr[r], o);
    }
    for (int off = L / 2; off > 0; off >>= 1) o += __shfl_xor(o, off, L);
    if (sub == 0) out[(t * H + h) * V + col] = o;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = sub * R + r;
    if (d < D) column[d] = S[r];
  }
}

template <typename T>
__global__ __launch_bounds__(PAE_WAVE) void delta_gated_norm_kernel(const float* __restrict__ o, const T* __restrict__ proj,
                                                                    int64_t row_stride, int gate_offset,
                                                                    const void* __restrict__ weight, int w_is_f32, float eps,
                                                                    int H, int V, T* __restrict__ out) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* x = o + (t * H + h) * V;
  float ss = 0.f;
  for (int i = lane; i < V; i += PAE_WAVE) ss = fmaf(x[i], x[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)V + eps);
  const T* gate = proj + t * row_stride + gate_offset + h * V;
  for (int i = lane; i < V; i += PAE_WAVE)
    out[(t * H + h) * V + i] = from_f32<T>(x[i] * inv * load_param(weight, w_is_f32, i) * silu_f(to_f32(gate[i])));
}

static int lanes_per_column(int D, int R) {
  int L = 1;
  while (L * R < D) L *= 2;
  return L;
}

extern "C" int pae_delta_rule_step(int dtype, const void* proj, int64_t row_stride, int num_tokens, int num_seqs,
                                   const int* tok_seq, const int* positions, const int* seq_runs, const int* slots,
                                   const float* conv_w, float* conv_tail, int64_t tail_slot_stride, int taps, int G,
                                   int H, int D, int V, const float* a_log, const float* dt_bias, float unit_eps,
                                   float* state, int64_t state_slot_stride, const void* norm_w, int w_is_f32,
                                   float norm_eps, float* work, void* out, hipStream_t stream) {
  PAE_REQUIRE(G > 0 && H > 0 && H % G == 0 && D > 0 && V > 0, "delta rule: bad head sizes G=%d H=%d D=%d V=%d", G, H, D, V);
  PAE_REQUIRE(taps >= 1 && taps <= 64, "delta rule: %d convolution taps", taps);
  PAE_REQUIRE(D <= 1024, "delta rule: key width %d exceeds 1024", D);
  PAE_REQUIRE(H <= 65535 && num_seqs <= 65535, "delta rule: %d heads, %d sequences exceed the grid", H, num_seqs);
  const int64_t C = 2 * (int64_t)G * D + (int64_t)H * V;
  PAE_REQUIRE(C * 4 <= 64 * 1024, "delta rule: %lld convolved channels exceed the kernel's 64 KB of LDS", (long long)C);
  PAE_REQUIRE(row_stride >= C + (int64_t)H * V + 2 * H, "delta rule: row stride %lld too small", (long long)row_stride);
  PAE_REQUIRE(dtype == PAE_F32 || dtype == PAE_BF16, "delta rule: unknown dtype code %d", dtype);
  if (num_tokens <= 0 || num_seqs <= 0) return 0;
  // work: q [T][G][D], k [T][G][D], v [T][H][V], beta [T][H], decay [T][H], o [T][H][V]
  float* q = work;
  float* k = q + (int64_t)num_tokens * G * D;
  float* v = k + (int64_t)num_tokens * G * D;
  float* beta = v + (int64_t)num_tokens * H * V;
  float* decay = beta + (int64_t)num_tokens * H;
  float* o = decay + (int64_t)num_tokens * H;
  const int4* runs = (const int4*)seq_runs;
  const int R = 16;
  const int L = lanes_per_column(D, R);
  dim3 tail_grid((unsigned)((C + 255) / 256), num_seqs);
  dim3 rec_grid((V + 256 / L - 1) / (256 / L), H, num_seqs);
  dim3 norm_grid(num_tokens, H);
#define DELTA_LAUNCH(T)                                                                                                 \
  delta_prepare_kernel<T><<<num_tokens, 256, (size_t)C * 4, stream>>>(                                                  \
      (const T*)proj, row_stride, tok_seq, positions, runs, slots, conv_w, conv_tail, tail_slot_stride, taps, G, H, D,  \
      V, a_log, dt_bias, unit_eps, q, k, v, beta, decay);                                                               \
  if (taps > 1)                                                                                                         \
    delta_conv_tail_kernel<T><<<tail_grid, 256, 0, stream>>>((const T*)proj, row_stride, runs, slots, conv_tail,        \
                                                             tail_slot_stride, taps, (int)C);                           \
  delta_recurrence_kernel<16><<<rec_grid, 256, 0, stream>>>(q, k, v, beta, decay, runs, slots, state,                   \
                                                            state_slot_stride, G, H, D, V, L, o);                       \
  delta_gated_norm_kernel<T><<<norm_grid, PAE_WAVE, 0, stream>>>(o, (const T*)proj, row_stride, (int)C, norm_w,         \
                                                                 w_is_f32, norm_eps, H, V, (T*)out)
  if (dtype == PAE_F32) {
    DELTA_LAUNCH(float);
  } else {
    DELTA_LAUNCH(bf16_t);
  }
#undef DELTA_LAUNCH
  return pae_check_launch("delta_rule_step");
}

// floats of `work` that pae_delta_rule_step needs for a step of `num_tokens` rows
extern "C" int64_t pae_delta_rule_work_floats(int num_tokens, int G, int H, int D, int V) {
  return (int64_t)num_tokens * (2 * (int64_t)G * D + 2 * (int64_t)H * V + 2 * H);
}
