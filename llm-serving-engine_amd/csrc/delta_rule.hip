// The gated delta rule and what stands around it: short causal convolutions over a request's tokens with their
// last inputs kept per request, the recurrence over a matrix state per head, and the gated norm of its read-out.
// Everything that enters the recurrence is float32; projections come in bfloat16 or float32.
#include "common.h"

// ---------------------------------------------------------------------------- short causal convolution + silu
// Request b brings the tokens [start[b], start[b + 1]) of the step.  For its token number i (from 0) and channel c
//   y[i, c] = silu(sum_j taps[c, j] * in(i - (width - 1) + j, c)),
// where in(n, c) is the step's own input for n >= 0 and, for n < 0, the request's kept input number width - 1 + n
// (window[slot, width - 1 + n, c]: the last width - 1 inputs of earlier steps, zeros at a request's start).
// One thread per (token, channel); the window is read here and written by the kernel below.
#define MAX_TAPS 16
template <typename T>
__global__ void causal_conv_kernel(const T* __restrict__ x, int x_stride, int channels, const float* __restrict__ taps,
                                   int width, const int* __restrict__ token_request, const int* __restrict__ start,
                                   const int* __restrict__ slots, const float* __restrict__ window, T* __restrict__ out) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int t = blockIdx.x, b = token_request[t];
  const int i = t - start[b];
  const float* kept = window ? window + (size_t)slots[b] * (width - 1) * channels : nullptr;
  float sum = 0.f;
  for (int j = 0; j < width; ++j) {
    const int n = i - (width - 1) + j;
    const float v = n >= 0 ? to_float(x[(size_t)(t - i + n) * x_stride + c]) : kept[(size_t)(width - 1 + n) * channels + c];
    sum += taps[(size_t)c * width + j] * v;
  }
  out[(size_t)t * channels + c] = from_float<T>(sum / (1.f + expf(-sum)));
}

// window[slot] <- the last width - 1 inputs after this step: the step's own last ones, and before them (for a step
// of fewer tokens) the kept ones moved up.  One thread per (request, channel) reads all it needs before it writes.
template <typename T>
__global__ void conv_window_kernel(const T* __restrict__ x, int x_stride, int channels, int width, const int* __restrict__ start,
                                   const int* __restrict__ slots, float* __restrict__ window) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int b = blockIdx.x, first = start[b], count = start[b + 1] - first;
  if (count <= 0) return;
  float* kept = window + (size_t)slots[b] * (width - 1) * channels;
  float next[MAX_TAPS];
#pragma unroll
  for (int i = 0; i < MAX_TAPS; ++i) {
    if (i < width - 1) {
      const int n = count - (width - 1) + i;  // the step's token number that lands at place i
      next[i] = n >= 0 ? to_float(x[(size_t)(first + n) * x_stride + c]) : kept[(size_t)(i + count) * channels + c];
    }
  }
#pragma unroll
  for (int i = 0; i < MAX_TAPS; ++i)
    if (i < width - 1) kept[(size_t)i * channels + c] = next[i];
}

extern "C" int llmserve_causal_conv(const void* x, int is_float, int tokens, int x_stride, int channels, const float* taps,
                                    int width, const int* token_request, const int* start, const int* slots, int requests,
                                    float* window, void* out, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (width < 1 || width > MAX_TAPS || channels < 1 || channels > x_stride || (width > 1 && !window)) return ERR_BAD_ARGUMENT;
  const int threads = channels <= 64 ? 64 : channels <= 128 ? 128 : 256;
  const dim3 grid(tokens, (channels + threads - 1) / threads);
  if (is_float)
    hipLaunchKernelGGL(causal_conv_kernel<float>, grid, dim3(threads), 0, stream, (const float*)x, x_stride, channels, taps, width,
                       token_request, start, slots, (const float*)window, (float*)out);
  else
    hipLaunchKernelGGL(causal_conv_kernel<bf16_t>, grid, dim3(threads), 0, stream, (const bf16_t*)x, x_stride, channels, taps,
                       width, token_request, start, slots, (const float*)window, (bf16_t*)out);
  if (width > 1) {
    const dim3 per_request(requests, (channels + threads - 1) / threads);
    if (is_float)
      hipLaunchKernelGGL(conv_window_kernel<float>, per_request, dim3(threads), 0, stream, (const float*)x, x_stride, channels,
                         width, start, slots, window);
    else
      hipLaunchKernelGGL(conv_window_kernel<bf16_t>, per_request, dim3(threads), 0, stream, (const bf16_t*)x, x_stride, channels,
                         width, start, slots, window);
  }
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- the recurrence
// A token's row of `mixed` is [q heads | k heads | v heads]: kv_heads of dim, kv_heads of dim, heads of vdim; value head h
// reads query/key head h / (heads / kv_heads).  `controls` [tokens, 2 heads] float32: b then a.  Per token and head
//   q <- q / sqrt(sum q^2 + 1e-6) * dim^-1/2,   k <- k / sqrt(sum k^2 + 1e-6),
//   beta = sigmoid(b),   g = exp(-exp(rate_h) * softplus(a + step_bias_h)),
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q            (S [dim, vdim], float32)
// Column j of S (the state of value dimension j) never meets another column.  A wave owns 16 columns of one (request,
// head): four neighbouring lanes share a column, each keeping a quarter of its rows (ROWS numbers) in registers for all
// the tokens of the request's step, and the two sums over a column's rows end with two exchanges between those lanes.
// The tokens are walked in runs of RUN: first the wave brings the run's q, k, v and controls from memory (all loads
// under way together: a token by itself would wait for memory every time), makes q and k unit vectors and the decays
// and betas (lane c those of the run's token c), and leaves them in LDS; then it walks the run token by token out of
// LDS and registers alone.  The state comes from state[slot, h] ([dim, vdim], columns side by side) and goes back there
// after the step's last token.
#define RUN 16
#define COLUMNS 16
template <typename T, int ROWS>  // 4 * ROWS >= dim; ROWS a multiple of 4
__global__ __launch_bounds__(64) void gated_delta_rule_kernel(const T* __restrict__ mixed, const float* __restrict__ controls,
                                                              const float* __restrict__ rate, const float* __restrict__ step_bias,
                                                              int heads, int kv_heads, int dim, int vdim,
                                                              const int* __restrict__ start, const int* __restrict__ slots,
                                                              float* __restrict__ state, float* __restrict__ out) {
  constexpr int PADDED = 4 * ROWS, PIECES = (PADDED + WAVE - 1) / WAVE, LINE = 4 * (ROWS + 4);  // (a quarter's rows, then 4 floats: banks)
  __shared__ __attribute__((aligned(16))) float keys[RUN][LINE], queries[RUN][LINE];
  __shared__ float decays[RUN], betas[RUN];
  const int b = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int column = blockIdx.z * COLUMNS + lane / 4, quarter = lane % 4;
  const bool owns = column < vdim;
  const int first = start[b], last = start[b + 1];
  if (last <= first) return;
  const int kv_head = head / (heads / kv_heads);
  const int row_width = 2 * kv_heads * dim + heads * vdim;
  float* mine = state + ((size_t)slots[b] * heads + head) * dim * vdim + column;
  float S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int i = quarter * ROWS + r;
    S[r] = (owns && i < dim) ? mine[(size_t)i * vdim] : 0.f;
  }
  const float speed = expf(rate[head]), bias = step_bias[head];
  const float q_scale = rsqrtf((float)dim);
  for (int t0 = first; t0 < last; t0 += RUN) {
    float q[RUN][PIECES], k[RUN][PIECES], v[RUN];
#pragma unroll
    for (int c = 0; c < RUN; ++c) {
      const bool valid = t0 + c < last;
      const T* row = mixed + (size_t)(valid ? t0 + c : t0) * row_width;
#pragma unroll
      for (int p = 0; p < PIECES; ++p) {
        const int i = p * WAVE + lane;
        q[c][p] = (valid && i < dim) ? to_float(row[kv_head * dim + i]) : 0.f;
        k[c][p] = (valid && i < dim) ? to_float(row[(kv_heads + kv_head) * dim + i]) : 0.f;
      }
      v[c] = (valid && owns) ? to_float(row[2 * kv_heads * dim + head * vdim + column]) : 0.f;
    }
    if (lane < RUN && t0 + lane < last) {
      const size_t at = (size_t)(t0 + lane) * 2 * heads;
      const float b_in = controls[at + head], a_in = controls[at + heads + head] + bias;
      const float softplus = a_in > 20.f ? a_in : log1pf(expf(a_in));
      betas[lane] = 1.f / (1.f + expf(-b_in));
      decays[lane] = expf(-speed * softplus);
    }
#pragma unroll
    for (int c = 0; c < RUN; ++c) {
      float q_squares = 0.f, k_squares = 0.f;
#pragma unroll
      for (int p = 0; p < PIECES; ++p) {
        q_squares += q[c][p] * q[c][p];
        k_squares += k[c][p] * k[c][p];
      }
      const float q_unit = q_scale / sqrtf(wave_sum(q_squares) + 1e-6f), k_unit = 1.f / sqrtf(wave_sum(k_squares) + 1e-6f);
#pragma unroll
      for (int p = 0; p < PIECES; ++p) {
        const int i = p * WAVE + lane;
        if (i < PADDED) {
          const int where = (i / ROWS) * (ROWS + 4) + i % ROWS;
          queries[c][where] = q[c][p] * q_unit;
          keys[c][where] = k[c][p] * k_unit;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < RUN; ++c) {
      if (t0 + c < last) {
        const float g = decays[c], beta = betas[c];
        const float4* key = (const float4*)&keys[c][quarter * (ROWS + 4)];
        const float4* query = (const float4*)&queries[c][quarter * (ROWS + 4)];
        float seen = 0.f;  // (g S)^T k, this lane's rows
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
          const float4 kk = key[r / 4];
          S[r] *= g; S[r + 1] *= g; S[r + 2] *= g; S[r + 3] *= g;
          seen += S[r] * kk.x; seen += S[r + 1] * kk.y; seen += S[r + 2] * kk.z; seen += S[r + 3] * kk.w;
        }
        seen += __shfl_xor(seen, 1, WAVE);
        seen += __shfl_xor(seen, 2, WAVE);
        const float u = beta * (v[c] - seen);
        float read = 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
          const float4 kk = key[r / 4], qq = query[r / 4];
          S[r] += kk.x * u; S[r + 1] += kk.y * u; S[r + 2] += kk.z * u; S[r + 3] += kk.w * u;
          read += S[r] * qq.x; read += S[r + 1] * qq.y; read += S[r + 2] * qq.z; read += S[r + 3] * qq.w;
        }
        read += __shfl_xor(read, 1, WAVE);
        read += __shfl_xor(read, 2, WAVE);
        if (owns && quarter == 0) out[(size_t)(t0 + c) * heads * vdim + head * vdim + column] = read;
      }
    }
    __syncthreads();  // the next run overwrites what this one read
  }
  if (owns) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int i = quarter * ROWS + r;
      if (i < dim) mine[(size_t)i * vdim] = S[r];
    }
  }
}

extern "C" int llmserve_gated_delta_rule(const void* mixed, int is_float, const float* controls, const float* rate,
                                         const float* step_bias, int heads, int kv_heads, int dim, int vdim, const int* start,
                                         const int* slots, int requests, float* state, float* out, hipStream_t stream) {
  if (requests <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads || dim < 1 || dim > 256 || vdim < 1 || heads > 65535) return ERR_BAD_ARGUMENT;
  const dim3 grid(requests, heads, (vdim + COLUMNS - 1) / COLUMNS);
#define LAUNCH_RULE(TYPE, ROWS)                                                                                              \
  hipLaunchKernelGGL((gated_delta_rule_kernel<TYPE, ROWS>), grid, dim3(WAVE), 0, stream, (const TYPE*)mixed, controls, rate, \
                     step_bias, heads, kv_heads, dim, vdim, start, slots, state, out)
  if (is_float) {
    if (dim <= 32) LAUNCH_RULE(float, 8); else if (dim <= 64) LAUNCH_RULE(float, 16); else if (dim <= 128) LAUNCH_RULE(float, 32); else LAUNCH_RULE(float, 64);
  } else {
    if (dim <= 32) LAUNCH_RULE(bf16_t, 8); else if (dim <= 64) LAUNCH_RULE(bf16_t, 16); else if (dim <= 128) LAUNCH_RULE(bf16_t, 32); else LAUNCH_RULE(bf16_t, 64);
  }
#undef LAUNCH_RULE
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- gated norm of the read-out
// out[t, h, :] = read[t, h, :] * rsqrt(mean(read[t, h, :]^2) + eps) * weight * silu(gates[t, gate_first + h * vdim + :]),
// one wave per (token, head).
template <typename T>
__global__ __launch_bounds__(64) void gated_head_norm_kernel(const float* __restrict__ read, const T* __restrict__ gates,
                                                             int gate_stride, int gate_first, const void* __restrict__ weight,
                                                             int weight_is_float, float eps, int vdim, T* __restrict__ out) {
  const size_t base = ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * vdim;
  const T* gate = gates + (size_t)blockIdx.x * gate_stride + gate_first + (size_t)blockIdx.y * vdim;
  float squares = 0.f;
  for (int i = threadIdx.x; i < vdim; i += WAVE) squares += read[base + i] * read[base + i];
  const float scale = rsqrtf(wave_sum(squares) / (float)vdim + eps);
  for (int i = threadIdx.x; i < vdim; i += WAVE) {
    const float z = to_float(gate[i]);
    out[base + i] = from_float<T>(read[base + i] * scale * load_as_float(weight, weight_is_float, i) * (z / (1.f + expf(-z))));
  }
}

extern "C" int llmserve_gated_head_norm(const float* read, const void* gates, int is_float, int gate_stride, int gate_first,
                                        const void* weight, int weight_is_float, float eps, int tokens, int heads, int vdim,
                                        void* out, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads < 1 || heads > 65535 || vdim < 1 || gate_first + heads * vdim > gate_stride) return ERR_BAD_ARGUMENT;
  const dim3 grid(tokens, heads);
  if (is_float)
    hipLaunchKernelGGL(gated_head_norm_kernel<float>, grid, dim3(WAVE), 0, stream, read, (const float*)gates, gate_stride, gate_first,
                       weight, weight_is_float, eps, vdim, (float*)out);
  else
    hipLaunchKernelGGL(gated_head_norm_kernel<bf16_t>, grid, dim3(WAVE), 0, stream, read, (const bf16_t*)gates, gate_stride,
                       gate_first, weight, weight_is_float, eps, vdim, (bf16_t*)out);
  return LAUNCH_STATUS();
}
