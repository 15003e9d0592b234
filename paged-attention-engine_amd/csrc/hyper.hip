// A residual stream kept as several copies (hyper-connections), with a scale per feature on every
// branch's output (layer scale), fused with the RMS norm that reads the stream next.
//
// The stream of a token is S rows x_0 .. x_{S-1} of `hidden` float32 numbers, stored one after the
// other.  A branch (mixer or feed-forward) that has produced y joins the stream by
//     x_t <- sum_s mix[s, t] x_s + out[t] * (ls * y)            (all t at once, from the old rows)
// and the next branch reads
//     u = sum_s in[s] x_s,    normed = u / sqrt(mean(u^2) + eps) * weight.
// One kernel does both for a token: it joins the branch that is pending (if any), writes the new
// rows back (unless only some rows are wanted, as for the logits), forms u and norms it.  With
// S = 1, mix = [[1]] and out = [1] this is the ordinary residual sum with a layer scale; with
// in = (1, .., 1) the read is the plain sum of the copies, which is what the model's last norm sees.
// Everything is float32; the normed row is rounded once, to the activations' storage type.
// `y` is the branch's output in that type, or float32 partial sums [parts][rows][hidden] of a
// product split over k, added here in order.
#include "common.h"
#include "api.h"

#define HYPER_MAX_STREAMS 8

template <typename T>
__global__ __launch_bounds__(256) void hyper_norm_kernel(
    float* __restrict__ streams, int S, const void* __restrict__ y, int parts, int64_t part_stride,
    const void* __restrict__ ls, int ls_is_f32, const float* __restrict__ mix, const float* __restrict__ outw,
    const float* __restrict__ inw, const void* __restrict__ weight, int w_is_f32, float eps,
    const int* __restrict__ rows, T* __restrict__ out, int hidden, int write_back) {
  extern __shared__ __attribute__((aligned(16))) float u_lds[];  // [hidden]: the row the norm reads
  __shared__ float s_mix[HYPER_MAX_STREAMS * HYPER_MAX_STREAMS], s_out[HYPER_MAX_STREAMS], s_in[HYPER_MAX_STREAMS];
  __shared__ float scratch[4];
  const int b = blockIdx.x;
  const int64_t t = rows ? rows[b] : b;
  if (threadIdx.x < S * S && y) s_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    if (y) s_out[threadIdx.x] = outw[threadIdx.x];
    s_in[threadIdx.x] = inw[threadIdx.x];
  }
  __syncthreads();
  float* x = streams + t * S * (int64_t)hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    float xs[HYPER_MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < HYPER_MAX_STREAMS; ++s) xs[s] = s < S ? x[(int64_t)s * hidden + i] : 0.f;
    if (y) {
      float yv;
      if (parts > 0) {
        yv = 0.f;
        for (int p = 0; p < parts; ++p) yv += ((const float*)y)[p * part_stride + t * hidden + i];
      } else {
        yv = to_f32(((const T*)y)[t * hidden + i]);
      }
      if (ls) yv *= load_param(ls, ls_is_f32, i);
      float xn[HYPER_MAX_STREAMS];
#pragma unroll
      for (int to = 0; to < HYPER_MAX_STREAMS; ++to) {
        if (to >= S) break;
        float v = 0.f;
        for (int s = 0; s < S; ++s) v = fmaf(s_mix[s * S + to], xs[s], v);
        xn[to] = fmaf(s_out[to], yv, v);
      }
#pragma unroll
      for (int s = 0; s < HYPER_MAX_STREAMS; ++s) {
        if (s >= S) break;
        xs[s] = xn[s];
        if (write_back) x[(int64_t)s * hidden + i] = xn[s];
      }
    }
    float u = 0.f;
#pragma unroll
    for (int s = 0; s < HYPER_MAX_STREAMS; ++s)
      if (s < S) u = fmaf(s_in[s], xs[s], u);
    u_lds[i] = u;
    ss = fmaf(u, u, ss);
  }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += 256)
    out[(int64_t)b * hidden + i] = from_f32<T>(u_lds[i] * inv * load_param(weight, w_is_f32, i));
}

// The same with four features a thread (16-byte loads and stores of the copies), for widths in multiples of four
// and as many copies as the template says; the order of adding per element is the scalar kernel's.
template <typename T, int S>
__global__ __launch_bounds__(256) void hyper_norm_vec_kernel(
    float* __restrict__ streams, const void* __restrict__ y, int parts, int64_t part_stride, const void* __restrict__ ls,
    int ls_is_f32, const float* __restrict__ mix, const float* __restrict__ outw, const float* __restrict__ inw,
    const void* __restrict__ weight, int w_is_f32, float eps, const int* __restrict__ rows, T* __restrict__ out, int hidden,
    int write_back) {
  extern __shared__ __attribute__((aligned(16))) float u_lds[];
  __shared__ float scratch[4];
  const int b = blockIdx.x;
  const int64_t t = rows ? rows[b] : b;
  float r_mix[S][S], r_out[S], r_in[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    r_in[s] = inw[s];
    r_out[s] = y ? outw[s] : 0.f;
#pragma unroll
    for (int to = 0; to < S; ++to) r_mix[s][to] = y ? mix[s * S + to] : 0.f;
  }
  float* x = streams + t * S * (int64_t)hidden;
  float ss = 0.f;
  for (int i = threadIdx.x * 4; i < hidden; i += 1024) {
    float4 xs[S];
#pragma unroll
    for (int s = 0; s < S; ++s) xs[s] = *reinterpret_cast<const float4*>(x + (int64_t)s * hidden + i);
    if (y) {
      float yv[4];
      if (parts > 0) {
        float4 sum = *reinterpret_cast<const float4*>((const float*)y + t * hidden + i);
        for (int p = 1; p < parts; ++p) {
          const float4 more = *reinterpret_cast<const float4*>((const float*)y + p * part_stride + t * hidden + i);
          sum.x += more.x; sum.y += more.y; sum.z += more.z; sum.w += more.w;
        }
        yv[0] = 0.f + sum.x; yv[1] = 0.f + sum.y; yv[2] = 0.f + sum.z; yv[3] = 0.f + sum.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[e] = to_f32(((const T*)y)[t * hidden + i + e]);
      }
      if (ls)
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[e] *= load_param(ls, ls_is_f32, i + e);
      float4 xn[S];
#pragma unroll
      for (int to = 0; to < S; ++to) {
        float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < S; ++s) {
          v[0] = fmaf(r_mix[s][to], xs[s].x, v[0]);
          v[1] = fmaf(r_mix[s][to], xs[s].y, v[1]);
          v[2] = fmaf(r_mix[s][to], xs[s].z, v[2]);
          v[3] = fmaf(r_mix[s][to], xs[s].w, v[3]);
        }
        xn[to] = make_float4(fmaf(r_out[to], yv[0], v[0]), fmaf(r_out[to], yv[1], v[1]), fmaf(r_out[to], yv[2], v[2]),
                             fmaf(r_out[to], yv[3], v[3]));
      }
#pragma unroll
      for (int s = 0; s < S; ++s) {
        xs[s] = xn[s];
        if (write_back) *reinterpret_cast<float4*>(x + (int64_t)s * hidden + i) = xn[s];
      }
    }
    float u[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < S; ++s) {
      u[0] = fmaf(r_in[s], xs[s].x, u[0]);
      u[1] = fmaf(r_in[s], xs[s].y, u[1]);
      u[2] = fmaf(r_in[s], xs[s].z, u[2]);
      u[3] = fmaf(r_in[s], xs[s].w, u[3]);
    }
    *reinterpret_cast<float4*>(u_lds + i) = make_float4(u[0], u[1], u[2], u[3]);
#pragma unroll
    for (int e = 0; e < 4; ++e) ss = fmaf(u[e], u[e], ss);
  }
  ss = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
  for (int i = threadIdx.x * 4; i < hidden; i += 1024) {
    const float4 u = *reinterpret_cast<const float4*>(u_lds + i);
    const float v[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) out[(int64_t)b * hidden + i + e] = from_f32<T>(v[e] * inv * load_param(weight, w_is_f32, i + e));
  }
}

extern "C" int pae_hyper_norm(int dtype, float* streams, int num_streams, const void* y, int parts, int64_t part_stride,
                              const void* ls, int ls_is_f32, const float* mix, const float* outw, const float* inw,
                              const void* weight, int w_is_f32, float eps, const int* rows, void* out, int num_rows,
                              int hidden, int write_back, hipStream_t stream) {
  PAE_REQUIRE(num_streams >= 1 && num_streams <= HYPER_MAX_STREAMS, "hyper_norm: %d copies of the stream (1..%d)", num_streams,
              HYPER_MAX_STREAMS);
  PAE_REQUIRE(num_rows >= 0 && hidden > 0 && hidden <= 16384, "hyper_norm: bad sizes rows=%d H=%d (widths up to 16,384)", num_rows, hidden);
  PAE_REQUIRE(parts >= 0, "hyper_norm: negative number of partial sums");
  PAE_REQUIRE(!y || (mix && outw), "hyper_norm: a pending branch needs its mix matrix and out weights");
  PAE_REQUIRE(inw && weight && out && streams, "hyper_norm: read weights, norm weight, stream and output are needed");
  PAE_REQUIRE(!(rows && write_back), "hyper_norm: a row gather may not write the stream back");
  if (num_rows == 0) return 0;
  const size_t lds = (size_t)hidden * sizeof(float);
#define HYPER_VEC(T, S)                                                                                              \
  hyper_norm_vec_kernel<T, S><<<num_rows, 256, lds, stream>>>(streams, y, parts, part_stride, ls, ls_is_f32, mix, outw, \
                                                             inw, weight, w_is_f32, eps, rows, (T*)out, hidden, write_back)
#define HYPER_VEC_BY_S(T)                        \
  switch (num_streams) {                         \
    case 1: HYPER_VEC(T, 1); break;              \
    case 2: HYPER_VEC(T, 2); break;              \
    case 3: HYPER_VEC(T, 3); break;              \
    default: HYPER_VEC(T, 4); break;             \
  }
  if (hidden % 4 == 0 && num_streams <= 4 && (dtype == PAE_F32 || dtype == PAE_BF16)) {
    if (dtype == PAE_F32) {
      HYPER_VEC_BY_S(float);
    } else {
      HYPER_VEC_BY_S(bf16_t);
    }
    return pae_check_launch("hyper_norm");
  }
#undef HYPER_VEC_BY_S
#undef HYPER_VEC
  if (dtype == PAE_F32)
    hyper_norm_kernel<float><<<num_rows, 256, lds, stream>>>(streams, num_streams, y, parts, part_stride, ls, ls_is_f32, mix,
                                                            outw, inw, weight, w_is_f32, eps, rows, (float*)out, hidden,
                                                            write_back);
  else if (dtype == PAE_BF16)
    hyper_norm_kernel<bf16_t><<<num_rows, 256, lds, stream>>>(streams, num_streams, y, parts, part_stride, ls, ls_is_f32, mix,
                                                             outw, inw, weight, w_is_f32, eps, rows, (bf16_t*)out, hidden,
                                                             write_back);
  else
    return pae_fail("hyper_norm: unknown dtype code %d", dtype);
  return pae_check_launch("hyper_norm");
}

// streams[t][s] = row t of `src` for every copy s: the start state of the copies (all equal to the
// embedding's output).
__global__ void hyper_spread_kernel(float* __restrict__ streams, const float* __restrict__ src, int S, int hidden) {
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = src[t * hidden + i];
    for (int s = 0; s < S; ++s) streams[(t * S + s) * hidden + i] = v;
  }
}

extern "C" int pae_hyper_spread(float* streams, const float* src, int num_rows, int num_streams, int hidden,
                                hipStream_t stream) {
  PAE_REQUIRE(num_rows >= 0 && num_streams >= 1 && hidden > 0, "hyper_spread: bad sizes rows=%d S=%d H=%d", num_rows,
              num_streams, hidden);
  if (num_rows == 0) return 0;
  hyper_spread_kernel<<<num_rows, 256, 0, stream>>>(streams, src, num_streams, hidden);
  return pae_check_launch("hyper_spread");
}

// out[t] = sum_s streams[t][s]: the stream as one row (for looking at it from outside).
__global__ void hyper_collapse_kernel(float* __restrict__ out, const float* __restrict__ streams, int S, int hidden) {
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = 0.f;
    for (int s = 0; s < S; ++s) v += streams[(t * S + s) * hidden + i];
    out[t * hidden + i] = v;
  }
}

extern "C" int pae_hyper_collapse(float* out, const float* streams, int num_rows, int num_streams, int hidden,
                                  hipStream_t stream) {
  PAE_REQUIRE(num_rows >= 0 && num_streams >= 1 && hidden > 0, "hyper_collapse: bad sizes rows=%d S=%d H=%d", num_rows,
              num_streams, hidden);
  if (num_rows == 0) return 0;
  hyper_collapse_kernel<<<num_rows, 256, 0, stream>>>(out, streams, num_streams, hidden);
  return pae_check_launch("hyper_collapse");
}
