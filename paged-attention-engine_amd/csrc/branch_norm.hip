// Kernels of blocks that normalise a branch's output instead of its input, and of the plain
// (ungated) feed-forward.
//
//   rows_from_residual   out[t] = T(residual[t]): the float32 stream as a product's operand
//   norm_scale_add       residual[t] += scale * y[t] / sqrt(mean(y[t]^2) + eps) * w, and optionally
//                        next[t] = T(residual[t]) for the product that reads the stream next
//   activation           x <- act(x) in place: 0 gelu by erf, 1 gelu by tanh, 2 silu
//
// Sums, the division and the residual are float32; `y` may come as the activation type or as
// float32 partial sums [parts][rows][hidden] of a product split along k, added here in order.
#include "common.h"
#include "api.h"

template <typename T>
__global__ void rows_from_residual_kernel(T* __restrict__ out, const float* __restrict__ residual, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(residual[i]);
}

extern "C" int pae_rows_from_residual(int dtype, void* out, const float* residual, int64_t n, hipStream_t stream) {
  if (n <= 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == PAE_F32)
    rows_from_residual_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, residual, n);
  else if (dtype == PAE_BF16)
    rows_from_residual_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, residual, n);
  else
    return pae_fail("rows_from_residual: unknown dtype code %d", dtype);
  return pae_check_launch("rows_from_residual");
}

template <typename T>
__device__ __forceinline__ float branch_at(const void* y, int parts, int64_t part_stride, int64_t idx) {
  if (parts == 0) return to_f32(((const T*)y)[idx]);
  float sum = 0.f;
  for (int p = 0; p < parts; ++p) sum += ((const float*)y)[p * part_stride + idx];
  return sum;
}

template <typename T>
__global__ __launch_bounds__(256) void norm_scale_add_kernel(float* __restrict__ residual, const void* __restrict__ y,
                                                             int parts, int64_t part_stride,
                                                             const void* __restrict__ weight, int w_is_f32, float eps,
                                                             float scale, T* __restrict__ next, int hidden) {
  extern __shared__ float held[];  // the row of y, when it fits
  __shared__ float scratch[4];
  const int64_t base = (int64_t)blockIdx.x * hidden;
  const bool keep = hidden <= 8192;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const float v = branch_at<T>(y, parts, part_stride, base + i);
    if (keep) held[i] = v;
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += 256) {
    const float v = keep ? held[i] : branch_at<T>(y, parts, part_stride, base + i);
    const float r = residual[base + i] + scale * (v * inv * load_param(weight, w_is_f32, i));
    residual[base + i] = r;
    if (next) next[base + i] = from_f32<T>(r);
  }
}

// Widths that are multiples of four up to 4,096: a thread owns up to four chunks of four columns, and
// everything it needs (the branch's row, the residual, the weight) is asked for at once, before the
// sum of squares is known: one trip to memory, then arithmetic, then the stores.
template <typename T>
__global__ __launch_bounds__(256) void norm_scale_add_vec_kernel(float* __restrict__ residual, const void* __restrict__ y,
                                                                 int parts, int64_t part_stride,
                                                                 const void* __restrict__ weight, int w_is_f32, float eps,
                                                                 float scale, T* __restrict__ next, int hidden) {
  __shared__ float scratch[4];
  const int64_t base = (int64_t)blockIdx.x * hidden;
  const int nvec = hidden / 4;
  float yv[4][4], rv[4][4], wv[4][4];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int v4 = threadIdx.x + 256 * c;
    if (v4 >= nvec) break;
    if (parts == 0) {
      if (sizeof(T) == 4) {
        const float4 a = reinterpret_cast<const float4*>((const float*)y + base)[v4];
        yv[c][0] = a.x; yv[c][1] = a.y; yv[c][2] = a.z; yv[c][3] = a.w;
      } else {
        const uint2 a = reinterpret_cast<const uint2*>((const bf16_t*)y + base)[v4];
        yv[c][0] = __uint_as_float(a.x << 16); yv[c][1] = __uint_as_float(a.x & 0xffff0000u);
        yv[c][2] = __uint_as_float(a.y << 16); yv[c][3] = __uint_as_float(a.y & 0xffff0000u);
      }
    } else {
      yv[c][0] = yv[c][1] = yv[c][2] = yv[c][3] = 0.f;
      for (int p = 0; p < parts; ++p) {  // partial sums are added in order
        const float4 a = reinterpret_cast<const float4*>((const float*)y + p * part_stride + base)[v4];
        yv[c][0] += a.x; yv[c][1] += a.y; yv[c][2] += a.z; yv[c][3] += a.w;
      }
    }
    const float4 r = reinterpret_cast<const float4*>(residual + base)[v4];
    rv[c][0] = r.x; rv[c][1] = r.y; rv[c][2] = r.z; rv[c][3] = r.w;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      wv[c][i] = load_param(weight, w_is_f32, 4 * v4 + i);
      ss = fmaf(yv[c][i], yv[c][i], ss);
    }
  }
  const float total = block_sum<4>(ss, scratch);
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int v4 = threadIdx.x + 256 * c;
    if (v4 >= nvec) break;
    float r[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = rv[c][i] + scale * (yv[c][i] * inv * wv[c][i]);
    reinterpret_cast<float4*>(residual + base)[v4] = make_float4(r[0], r[1], r[2], r[3]);
    if (next) {
      if (sizeof(T) == 4) {
        reinterpret_cast<float4*>((float*)next + base)[v4] = make_float4(r[0], r[1], r[2], r[3]);
      } else {
        bf16_t h[4] = {__float2bfloat16(r[0]), __float2bfloat16(r[1]), __float2bfloat16(r[2]), __float2bfloat16(r[3])};
        reinterpret_cast<uint2*>((bf16_t*)next + base)[v4] = *reinterpret_cast<const uint2*>(h);
      }
    }
  }
}

extern "C" int pae_norm_scale_add(int dtype, float* residual, const void* y, int parts, int64_t part_stride,
                                  const void* weight, int w_is_f32, float eps, float scale, void* next, int num_rows,
                                  int hidden, hipStream_t stream) {
  PAE_REQUIRE(parts >= 0 && num_rows >= 0 && hidden > 0, "norm_scale_add: bad sizes rows=%d H=%d parts=%d", num_rows,
              hidden, parts);
  if (num_rows == 0) return 0;
  const size_t lds = hidden <= 8192 ? (size_t)hidden * sizeof(float) : 0;
  if (hidden % 4 == 0 && hidden <= 4096 && part_stride % 4 == 0 && (dtype == PAE_F32 || dtype == PAE_BF16)) {
    if (dtype == PAE_F32)
      norm_scale_add_vec_kernel<float><<<num_rows, 256, 0, stream>>>(residual, y, parts, part_stride, weight, w_is_f32,
                                                                     eps, scale, (float*)next, hidden);
    else
      norm_scale_add_vec_kernel<bf16_t><<<num_rows, 256, 0, stream>>>(residual, y, parts, part_stride, weight, w_is_f32,
                                                                      eps, scale, (bf16_t*)next, hidden);
    return pae_check_launch("norm_scale_add");
  }
  if (dtype == PAE_F32)
    norm_scale_add_kernel<float><<<num_rows, 256, lds, stream>>>(residual, y, parts, part_stride, weight, w_is_f32, eps,
                                                                 scale, (float*)next, hidden);
  else if (dtype == PAE_BF16)
    norm_scale_add_kernel<bf16_t><<<num_rows, 256, lds, stream>>>(residual, y, parts, part_stride, weight, w_is_f32,
                                                                  eps, scale, (bf16_t*)next, hidden);
  else
    return pae_fail("norm_scale_add: unknown dtype code %d", dtype);
  return pae_check_launch("norm_scale_add");
}

template <typename T>
__global__ void activation_kernel(T* __restrict__ x, int64_t n, int kind) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = from_f32<T>(act_of(to_f32(x[i]), kind));
}

// eight bfloat16 numbers a thread (one 16-byte load and store), for sizes that are multiples of eight
__global__ void activation_bf16x8_kernel(uint4* __restrict__ x, int64_t nvec, int kind) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= nvec) return;
  uint4 v = x[i];
  unsigned* w = reinterpret_cast<unsigned*>(&v);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const bf16_t lo = __float2bfloat16(act_of(__uint_as_float(w[j] << 16), kind));
    const bf16_t hi = __float2bfloat16(act_of(__uint_as_float(w[j] & 0xffff0000u), kind));
    w[j] = (unsigned)*reinterpret_cast<const unsigned short*>(&lo) | ((unsigned)*reinterpret_cast<const unsigned short*>(&hi) << 16);
  }
  x[i] = v;
}

extern "C" int pae_activation(int dtype, void* x, int64_t n, int kind, hipStream_t stream) {
  PAE_REQUIRE(kind >= 0 && kind <= 2, "activation: unknown kind %d", kind);
  if (n <= 0) return 0;
  if (dtype == PAE_BF16 && n % 8 == 0 && (uintptr_t)x % 16 == 0) {
    activation_bf16x8_kernel<<<(unsigned)((n / 8 + 255) / 256), 256, 0, stream>>>((uint4*)x, n / 8, kind);
    return pae_check_launch("activation");
  }
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == PAE_F32)
    activation_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, n, kind);
  else if (dtype == PAE_BF16)
    activation_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, n, kind);
  else
    return pae_fail("activation: unknown dtype code %d", dtype);
  return pae_check_launch("activation");
}
