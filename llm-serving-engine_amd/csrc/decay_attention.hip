// Linear attention over a matrix state per head that fades by a fixed factor a token:
//   S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   S [dim, vdim] float32 per (request, head),
// with q, k, v = act of columns of a projected row.  Compiled once per query/key size (-DHEAD_DIM=...).
//
// Two kernels.  `decay_attention_runs` walks a request's tokens in runs of 16 on the matrix cores in true float32
// (v_mfma_f32_16x16x4_f32); over a run of n tokens that starts from the state S,
//   o_t = decay^(t+1) S^T q_t + sum_(s <= t) decay^(t-s) (q_t . k_s) v_s        (t, s count from 0 inside the run)
//   S  <- decay^n S + sum_(s < n) decay^(n-1-s) k_s v_s^T.
// A wave owns 16 value columns of one (request, head) and all of S's rows for them, as accumulator tiles:
//   P^T[s][t] = K Q^T       A = K rows, B = Q rows; the lane that holds P^T[s = 4g + e][t = i] scales it by decay^(t-s)
//   O[t][v]   = P V         the accumulator of P^T is, as it lies, the A operand P (row t = i, contraction s = 4g + e)
//   O[t][v]  += (decay^(t+1) Q) S     the accumulator tiles of S are, as they lie, the B operand (contraction over S's rows)
//   S[d][v]   = decay^n S + (decay^(n-1-s) K)^T V    A = K read across (rows of K^T), B = V as above
// so nothing passes between lanes.  Sizes that are no multiple of 16, and steps of very few tokens a request
// (decoding), go to `decay_attention_tokens`: a workgroup owns 64 value columns of one (request, head), its four
// waves deal S's rows out among them and keep them in registers, token by token; the waves' shares of o are added
// through LDS in wave order.  Either way the state is read once and written once a step, and a value depends only
// on its own request's tokens.
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<query/key size>"
#endif
#if HEAD_DIM < 1 || HEAD_DIM > 512
#error "HEAD_DIM must lie between 1 and 512"
#endif

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int D = HEAD_DIM;
constexpr int RUN = 16;

template <bool SILU>
__device__ __forceinline__ float activated(float z) {
  return SILU ? z / (1.f + expf(-z)) : z;
}

struct DecaySizes {
  int x_width, q_first, k_first, v_first, heads, vdim;
};

#if HEAD_DIM % 16 == 0
constexpr int D_TILES = D / 16;

__device__ __forceinline__ f32x4 load_four(const float* p) { return *(const f32x4*)p; }
__device__ __forceinline__ f32x4 load_four(const bf16_t* p) {
  const uint2 raw = *(const uint2*)p;  // a bfloat16 is the upper half of the float32 of the same value
  return (f32x4){__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                 __uint_as_float(raw.y & 0xffff0000u)};
}

// grid (vdim / 16, heads, requests), one wave a workgroup
template <typename T, bool SILU>
__global__ __launch_bounds__(64) void decay_attention_runs_kernel(const T* __restrict__ x, DecaySizes z,
                                                                  const float* __restrict__ decays,
                                                                  const int* __restrict__ query_start,
                                                                  const int* __restrict__ state_slots, float* __restrict__ state,
                                                                  float* __restrict__ out) {
  __shared__ float power[RUN + 1];
  const int v0 = blockIdx.x * 16, head = blockIdx.y, request = blockIdx.z;
  const int lane = threadIdx.x, i = lane & 15, g = lane >> 4;
  const int begin = query_start[request], end = query_start[request + 1];
  if (begin >= end) return;  // a request that only pads a captured step
  if (lane <= RUN) {
    double p = 1.0;
    for (int j = 0; j < lane; ++j) p *= (double)decays[head];
    power[lane] = (float)p;
  }
  __syncthreads();
  // S[d][v] of this wave's columns: lane (i, g) holds rows 16 tile + 4 g + e of column v0 + i
  float* s_at = state + (((size_t)state_slots[request] * z.heads + head) * D + 4 * g) * z.vdim + v0 + i;
  f32x4 S[D_TILES];
#pragma unroll
  for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
    for (int e = 0; e < 4; ++e) S[tile][e] = s_at[(size_t)(16 * tile + e) * z.vdim];
  const int out_width = z.heads * z.vdim;

  for (int t0 = begin; t0 < end; t0 += RUN) {
    const int n = min(RUN, end - t0);
    // Q and K by rows: lane (i, g) holds d = 16 tile + 4 g .. + 3 of token i (a token beyond the run counts as zeros)
    const bool live = i < n;
    const T* mine = x + (size_t)(t0 + min(i, n - 1)) * z.x_width + head * D + 4 * g;
    f32x4 q[D_TILES], k[D_TILES];
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile) {
      q[tile] = load_four(mine + z.q_first + 16 * tile);
      k[tile] = load_four(mine + z.k_first + 16 * tile);
    }
    // V, and K read across: lane (i, g) holds column i of tokens 4 g + e
    f32x4 v, across[D_TILES];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const T* theirs = x + (size_t)(t0 + min(4 * g + e, n - 1)) * z.x_width;
      v[e] = to_float(theirs[z.v_first + head * z.vdim + v0 + i]);
#pragma unroll
      for (int tile = 0; tile < D_TILES; ++tile) across[tile][e] = to_float(theirs[z.k_first + head * D + 16 * tile + i]);
    }
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        q[tile][e] = live ? activated<SILU>(q[tile][e]) : 0.f;
        k[tile][e] = live ? activated<SILU>(k[tile][e]) : 0.f;
      }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int s = 4 * g + e;
      v[e] = s < n ? activated<SILU>(v[e]) : 0.f;
      const float fade = s < n ? power[n - 1 - s] : 0.f;
#pragma unroll
      for (int tile = 0; tile < D_TILES; ++tile) across[tile][e] = s < n ? activated<SILU>(across[tile][e]) * fade : 0.f;
    }
    // P^T[s][t] = k_s . q_t, faded by decay^(t - s) where s <= t
    f32x4 p = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) p = __builtin_amdgcn_mfma_f32_16x16x4f32(k[tile][e], q[tile][e], p, 0, 0, 0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int s = 4 * g + e;
      p[e] = s <= i ? p[e] * power[i - s] : 0.f;
    }
    // O[t][v] = sum_s P[t][s] V[s][v] + sum_d decay^(t+1) Q[t][d] S[d][v]
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < 4; ++e) o = __builtin_amdgcn_mfma_f32_16x16x4f32(p[e], v[e], o, 0, 0, 0);
    const float carried = power[i + 1];
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) o = __builtin_amdgcn_mfma_f32_16x16x4f32(q[tile][e] * carried, S[tile][e], o, 0, 0, 0);
    // S = decay^n S + sum_s decay^(n-1-s) k_s v_s^T
    const float whole = power[n];
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile) {
#pragma unroll
      for (int e = 0; e < 4; ++e) S[tile][e] *= whole;
#pragma unroll
      for (int e = 0; e < 4; ++e) S[tile] = __builtin_amdgcn_mfma_f32_16x16x4f32(across[tile][e], v[e], S[tile], 0, 0, 0);
    }
    // lane (i, g) holds O[t = 4 g + e][v0 + i]
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (4 * g + e < n) out[(size_t)(t0 + 4 * g + e) * out_width + head * z.vdim + v0 + i] = o[e];
  }
#pragma unroll
  for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
    for (int e = 0; e < 4; ++e) s_at[(size_t)(16 * tile + e) * z.vdim] = S[tile][e];
}
#endif

// grid (ceil(vdim / 64), heads, requests), four waves: lane = value column, wave w owns S's rows w, w + 4, ...
constexpr int TOKEN_WAVES = 4;
constexpr int ROWS = (D + TOKEN_WAVES - 1) / TOKEN_WAVES;

template <typename T, bool SILU>
__global__ __launch_bounds__(TOKEN_WAVES * 64) void decay_attention_tokens_kernel(const T* __restrict__ x, DecaySizes z,
                                                                                  const float* __restrict__ decays,
                                                                                  const int* __restrict__ query_start,
                                                                                  const int* __restrict__ state_slots,
                                                                                  float* __restrict__ state, float* __restrict__ out) {
  __shared__ float asked[D], keyed[D];
  __shared__ float shares[TOKEN_WAVES][64];
  const int head = blockIdx.y, request = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int column = blockIdx.x * 64 + lane;
  const bool live = column < z.vdim;
  const int begin = query_start[request], end = query_start[request + 1];
  if (begin >= end) return;
  const float decay = decays[head];
  float* s_at = state + ((size_t)state_slots[request] * z.heads + head) * D * z.vdim + min(column, z.vdim - 1);
  float S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = wave + TOKEN_WAVES * r;
    S[r] = live && d < D ? s_at[(size_t)d * z.vdim] : 0.f;
  }
  const int out_width = z.heads * z.vdim;
  for (int t = begin; t < end; ++t) {
    const T* row = x + (size_t)t * z.x_width;
    for (int e = threadIdx.x; e < D; e += blockDim.x) {
      asked[e] = activated<SILU>(to_float(row[z.q_first + head * D + e]));
      keyed[e] = activated<SILU>(to_float(row[z.k_first + head * D + e]));
    }
    const float value = live ? activated<SILU>(to_float(row[z.v_first + head * z.vdim + column])) : 0.f;
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int d = wave + TOKEN_WAVES * r;
      if (d < D) {
        S[r] = fmaf(decay, S[r], keyed[d] * value);
        o = fmaf(S[r], asked[d], o);
      }
    }
    shares[wave][lane] = o;
    __syncthreads();  // (also: everybody has read this token's q and k before the next token's are written)
    if (wave == 0 && live) {
      float sum = shares[0][lane];
#pragma unroll
      for (int w = 1; w < TOKEN_WAVES; ++w) sum += shares[w][lane];
      out[(size_t)t * out_width + head * z.vdim + column] = sum;
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int d = wave + TOKEN_WAVES * r;
    if (live && d < D) s_at[(size_t)d * z.vdim] = S[r];
  }
}

extern "C" int llmserve_decay_attention_head_dim() { return D; }

// x [tokens, x_width] (bfloat16 or float32) holds the heads' q and k (of HEAD_DIM) and v (of vdim) from the columns
// q_first, k_first, v_first; activation 0 none, 1 silu; decays float32 [heads]; query_start int32 [requests + 1];
// state_slots int32 [requests]; state float32 [slots, heads, HEAD_DIM, vdim]; out float32 [tokens, heads * vdim].
// `longest` is the most tokens a request of the step brings (or may bring, in a step that is replayed).
extern "C" int llmserve_decay_attention(const void* x, int is_float, int tokens, int x_width, int q_first, int k_first, int v_first,
                                        int heads, int vdim, int activation, const float* decays, const int* query_start,
                                        const int* state_slots, int requests, int longest, float* state, float* out,
                                        hipStream_t stream) {
  if (tokens <= 0 || requests <= 0) return 0;
  if (heads < 1 || heads > 65535 || requests > 65535 || vdim < 1 || activation < 0 || activation > 1 || q_first < 0 || k_first < 0 ||
      v_first < 0 || q_first + heads * D > x_width || k_first + heads * D > x_width || v_first + heads * vdim > x_width)
    return ERR_BAD_ARGUMENT;
  const DecaySizes z = {x_width, q_first, k_first, v_first, heads, vdim};
#define LAUNCH_DECAY(KERNEL, GRID, THREADS)                                                                                     \
  do {                                                                                                                          \
    if (is_float && activation)                                                                                                 \
      hipLaunchKernelGGL((KERNEL<float, true>), GRID, dim3(THREADS), 0, stream, (const float*)x, z, decays, query_start,         \
                         state_slots, state, out);                                                                              \
    else if (is_float)                                                                                                          \
      hipLaunchKernelGGL((KERNEL<float, false>), GRID, dim3(THREADS), 0, stream, (const float*)x, z, decays, query_start,        \
                         state_slots, state, out);                                                                              \
    else if (activation)                                                                                                        \
      hipLaunchKernelGGL((KERNEL<bf16_t, true>), GRID, dim3(THREADS), 0, stream, (const bf16_t*)x, z, decays, query_start,       \
                         state_slots, state, out);                                                                              \
    else                                                                                                                        \
      hipLaunchKernelGGL((KERNEL<bf16_t, false>), GRID, dim3(THREADS), 0, stream, (const bf16_t*)x, z, decays, query_start,      \
                         state_slots, state, out);                                                                              \
  } while (0)
#if HEAD_DIM % 16 == 0
  // (the rows' loads in the kernel of runs are 16 bytes wide in float32 and 8 in bfloat16: the columns begin accordingly)
  const int aligned = is_float ? 4 : 4;
  if (longest > 3 && vdim % 16 == 0 && x_width % aligned == 0 && q_first % aligned == 0 && k_first % aligned == 0) {
    LAUNCH_DECAY(decay_attention_runs_kernel, dim3(vdim / 16, heads, requests), 64);
    return LAUNCH_STATUS();
  }
#endif
  LAUNCH_DECAY(decay_attention_tokens_kernel, dim3((vdim + 63) / 64, heads, requests), TOKEN_WAVES * 64);
#undef LAUNCH_DECAY
  return LAUNCH_STATUS();
}
