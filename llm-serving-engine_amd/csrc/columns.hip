// Operations on rows and on runs of their columns: RMS norm of a run of columns, rotary tables with a magnitude,
// rotation of a run of columns per head, two streams side by side, an activation, and a gated add.  All arithmetic
// is float32; inputs and outputs are bfloat16 or float32.
#include "common.h"

#define ACT_SILU 0
#define ACT_GELU 1
#define ACT_GELU_TANH 2
#define ACT_RELU 3

__device__ __forceinline__ float activation_of(int activation, float z) {
  switch (activation) {
    case ACT_GELU: return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
    case ACT_GELU_TANH: return 0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
    case ACT_RELU: return fmaxf(z, 0.f);
    default: return z / (1.f + expf(-z));
  }
}

// ---------------------------------------------------------------------------- RMS norm of a run of columns
// out[t, out_first + c * copy_stride + i] = x[t, first + i] * rsqrt(mean_i(x[t, first + i]^2) + eps) * weight[i] for
// every copy c: a projection's output holds several vectors side by side, each with a norm of its own, and
// the normed vector may be wanted in several places of a wider row.
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_columns_kernel(const T* __restrict__ x, int x_stride, int first, int width,
                                                               const void* __restrict__ weight, int weight_is_float, float eps,
                                                               T* __restrict__ out, int out_stride, int out_first, int copies,
                                                               int copy_stride) {
  __shared__ float shared[17];
  const T* row = x + (size_t)blockIdx.x * x_stride + first;
  float squares = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = to_float(row[i]);
    squares += v * v;
  }
  const float scale = rsqrtf(block_sum(squares, shared) / (float)width + eps);
  T* dst = out + (size_t)blockIdx.x * out_stride + out_first;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const T value = from_float<T>(to_float(row[i]) * scale * load_as_float(weight, weight_is_float, i));
    for (int c = 0; c < copies; ++c) dst[(size_t)c * copy_stride + i] = value;
  }
}

extern "C" int llmserve_rms_norm_columns(const void* x, int is_float, int rows, int x_stride, int first, int width,
                                         const void* weight, int weight_is_float, float eps, void* out, int out_stride,
                                         int out_first, int copies, int copy_stride, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (width <= 0 || first < 0 || first + width > x_stride || copies < 1 ||
      out_first + (copies - 1) * copy_stride + width > out_stride)
    return ERR_BAD_ARGUMENT;
  const int threads = width <= 64 ? 64 : width <= 128 ? 128 : 256;
  if (is_float)
    hipLaunchKernelGGL(rms_norm_columns_kernel<float>, dim3(rows), dim3(threads), 0, stream, (const float*)x, x_stride, first,
                       width, weight, weight_is_float, eps, (float*)out, out_stride, out_first, copies, copy_stride);
  else
    hipLaunchKernelGGL(rms_norm_columns_kernel<bf16_t>, dim3(rows), dim3(threads), 0, stream, (const bf16_t*)x, x_stride, first,
                       width, weight, weight_is_float, eps, (bf16_t*)out, out_stride, out_first, copies, copy_stride);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- rotary table with a magnitude
// table[t][j] = magnitude * (cos, sin) of positions[t] * frequency[j], in float32.
__global__ void rotary_table_scaled_kernel(const int* __restrict__ positions, const float* __restrict__ frequency,
                                           float2* __restrict__ table, int half, float magnitude) {
  const float position = (float)positions[blockIdx.x];
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    float sine, cosine;
    sincosf(position * frequency[j], &sine, &cosine);
    table[(size_t)blockIdx.x * half + j] = make_float2(cosine * magnitude, sine * magnitude);
  }
}

extern "C" int llmserve_rotary_table_scaled(const int* positions, const float* frequency, float* table, int tokens, int half,
                                            float magnitude, hipStream_t stream) {
  if (tokens <= 0) return 0;
  hipLaunchKernelGGL(rotary_table_scaled_kernel, dim3(tokens), dim3(64), 0, stream, positions, frequency, (float2*)table, half,
                     magnitude);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- rotation of a run of columns per head
// For every head h: the `width` columns of x from first + h * head_stride go to the columns of out from out_first +
// h * out_head_stride; of them the first `dims` are rotated in adjacent pairs, (u, v) at columns (2i, 2i + 1) becoming
// (u cos_i - v sin_i, v cos_i + u sin_i) with the token's table entry i; the others are copied.
template <typename T>
__global__ void rotate_columns_kernel(const T* __restrict__ x, int x_stride, int first, int head_stride, int heads, int width,
                                      const float2* __restrict__ table, int dims, T* __restrict__ out, int out_stride,
                                      int out_first, int out_head_stride) {
  const T* row = x + (size_t)blockIdx.x * x_stride + first;
  T* dst = out + (size_t)blockIdx.x * out_stride + out_first;
  const float2* angles = table + (size_t)blockIdx.x * (dims / 2);
  for (int e = threadIdx.x; e < heads * width; e += blockDim.x) {
    const int head = e / width, c = e % width;
    const T* from = row + (size_t)head * head_stride;
    float value = to_float(from[c]);
    if (c < dims) {
      const float2 turn = angles[c / 2];
      const float other = to_float(from[c ^ 1]);
      value = (c & 1) ? value * turn.x + other * turn.y : value * turn.x - other * turn.y;
    }
    dst[(size_t)head * out_head_stride + c] = from_float<T>(value);
  }
}

extern "C" int llmserve_rotate_columns(const void* x, int is_float, int tokens, int x_stride, int first, int head_stride,
                                       int heads, int width, const float* table, int dims, void* out, int out_stride,
                                       int out_first, int out_head_stride, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (dims % 2 || dims > width || heads < 1 || first + (heads - 1) * head_stride + width > x_stride ||
      out_first + (heads - 1) * out_head_stride + width > out_stride)
    return ERR_BAD_ARGUMENT;
  const int threads = heads * width <= 64 ? 64 : heads * width <= 128 ? 128 : 256;
  if (is_float)
    hipLaunchKernelGGL(rotate_columns_kernel<float>, dim3(tokens), dim3(threads), 0, stream, (const float*)x, x_stride, first,
                       head_stride, heads, width, (const float2*)table, dims, (float*)out, out_stride, out_first, out_head_stride);
  else
    hipLaunchKernelGGL(rotate_columns_kernel<bf16_t>, dim3(tokens), dim3(threads), 0, stream, (const bf16_t*)x, x_stride, first,
                       head_stride, heads, width, (const float2*)table, dims, (bf16_t*)out, out_stride, out_first, out_head_stride);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- two streams side by side
// out[t] = [hidden[t] + delta[0][t] + delta[1][t] + ... | other[t]] in the output type: the operand of a product over both.
template <typename TO>
__global__ void join_rows_kernel(const float* __restrict__ hidden, const float* __restrict__ delta, int parts,
                                 size_t part_stride, const float* __restrict__ other, TO* __restrict__ out, int width) {
  const size_t base = (size_t)blockIdx.x * width;
  TO* dst = out + 2 * base;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = hidden[base + i];
    if (delta)
      for (int p = 0; p < parts; ++p) v += delta[p * part_stride + base + i];
    dst[i] = from_float<TO>(v);
    dst[width + i] = from_float<TO>(other[base + i]);
  }
}

extern "C" int llmserve_join_rows(const float* hidden, const float* delta, int parts, const float* other, void* out,
                                  int out_is_float, int rows, int width, hipStream_t stream) {
  if (rows <= 0) return 0;
  const size_t part_stride = (size_t)rows * width;
  if (out_is_float)
    hipLaunchKernelGGL(join_rows_kernel<float>, dim3(rows), dim3(256), 0, stream, hidden, delta, parts, part_stride, other,
                       (float*)out, width);
  else
    hipLaunchKernelGGL(join_rows_kernel<bf16_t>, dim3(rows), dim3(256), 0, stream, hidden, delta, parts, part_stride, other,
                       (bf16_t*)out, width);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- activation
template <typename T>
__global__ void activate_kernel(const T* __restrict__ in, T* __restrict__ out, size_t count, int activation) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
    out[i] = from_float<T>(activation_of(activation, to_float(in[i])));
}

extern "C" int llmserve_activate(const void* in, void* out, int is_float, int rows, int width, int activation,
                                 hipStream_t stream) {
  const size_t count = (size_t)rows * width;
  if (count == 0) return 0;
  const int blocks = (int)((count + 255) / 256 < 4096 ? (count + 255) / 256 : 4096);
  if (is_float)
    hipLaunchKernelGGL(activate_kernel<float>, dim3(blocks), dim3(256), 0, stream, (const float*)in, (float*)out, count, activation);
  else
    hipLaunchKernelGGL(activate_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (const bf16_t*)in, (bf16_t*)out, count, activation);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- gated add
// target[t] += sigmoid(gates[t, column]) * rows[t], all float32.
__global__ void add_gated_rows_kernel(float* __restrict__ target, const float* __restrict__ rows, const float* __restrict__ gates,
                                      int gate_stride, int column, int width) {
  const float gate = 1.f / (1.f + expf(-gates[(size_t)blockIdx.x * gate_stride + column]));
  const size_t base = (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) target[base + i] += gate * rows[base + i];
}

extern "C" int llmserve_add_gated_rows(float* target, const float* rows, const float* gates, int gate_stride, int column,
                                       int count, int width, hipStream_t stream) {
  if (count <= 0) return 0;
  if (column < 0 || column >= gate_stride) return ERR_BAD_ARGUMENT;
  hipLaunchKernelGGL(add_gated_rows_kernel, dim3(count), dim3(256), 0, stream, target, rows, gates, gate_stride, column, width);
  return LAUNCH_STATUS();
}
