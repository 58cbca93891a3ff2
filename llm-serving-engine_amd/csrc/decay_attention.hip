// Linear attention over a matrix state per head that fades by a fixed factor a token:
//   S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,   S [dim, vdim] float32 per (request, head),
// with q, k, v = act of columns of a projected row.  Compiled once per query/key size (-DHEAD_DIM=...).
//
// `decay_attention_runs` walks a request's tokens in runs of 16 on the matrix cores in true float32
// (v_mfma_f32_16x16x4_f32); over a run of n tokens that starts from the state S,
//   o_t = decay^(t+1) S^T q_t + sum_(s <= t) decay^(t-s) (q_t . k_s) v_s        (t, s count from 0 inside the run)
//   S  <- decay^n S + sum_(s < n) decay^(n-1-s) k_s v_s^T.
// A wave owns 16 value columns of one (request, head) and all of S's rows for them, as accumulator tiles:
//   P^T[s][t] = K Q^T       A = K rows, B = Q rows; the lane that holds P^T[s = 4g + e][t = i] scales it by decay^(t-s)
//   O[t][v]   = P V         the accumulator of P^T is, as it lies, the A operand P (row t = i, contraction s = 4g + e)
//   O[t][v]  += (decay^(t+1) Q) S     the accumulator tiles of S are, as they lie, the B operand (contraction over S's rows)
//   S[d][v]   = decay^n S + (decay^(n-1-s) K)^T V    A = K read across (rows of K^T), B = V as above
// so nothing passes between lanes.  The next run's operands are asked for before this run is computed.  A long
// portion is cut into segments that are walked side by side, each from an empty state; a second kernel hands the states
// on from segment to segment (F_j = decay^tokens F_(j-1) + the segment's own), and a third adds to a segment's tokens what
// they read of the state the segment starts from (decay^(t+1) q_t S_in): a 2,048-token portion is sixteen walks of eight
// runs instead of one of 128.  Sizes that are no multiple of 16, and steps of very few tokens a request
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

// The same by the hardware's exponential and reciprocal (an ulp or so each): the kernel of runs activates a hundred
// values a lane a run, and the exact forms' instructions were most of its time.
template <bool SILU>
__device__ __forceinline__ float activated_fast(float z) {
  return SILU ? z * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(z * -1.44269504088896f)) : z;
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

// base^n in float64 by squaring
__device__ __forceinline__ double whole_power(double base, int n) {
  double result = 1.0;
  for (; n > 0; n >>= 1, base *= base)
    if (n & 1) result *= base;
  return result;
}

// What a lane holds of a run of up to 16 tokens, as loaded (not yet activated): Q and K by rows (lane (i, g): d = 16
// tile + 4 g .. + 3 of token i), and V (of each of the wave's VT tiles of 16 columns) and K read across (lane (i, g):
// column i of tokens 4 g + e).
template <int VT>
struct RunOperands {
  f32x4 q[D_TILES], k[D_TILES], across[D_TILES], v[VT];
};

template <typename T, int VT>
__device__ __forceinline__ void load_run(RunOperands<VT>& r, const T* __restrict__ x, const DecaySizes& z, int head, int v0, int t0,
                                         int n, int i, int g) {
  const T* mine = x + (size_t)(t0 + min(i, n - 1)) * z.x_width + head * D + 4 * g;
#pragma unroll
  for (int tile = 0; tile < D_TILES; ++tile) {
    r.q[tile] = load_four(mine + z.q_first + 16 * tile);
    r.k[tile] = load_four(mine + z.k_first + 16 * tile);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const T* theirs = x + (size_t)(t0 + min(4 * g + e, n - 1)) * z.x_width;
#pragma unroll
    for (int j = 0; j < VT; ++j) r.v[j][e] = to_float(theirs[z.v_first + head * z.vdim + v0 + 16 * j + i]);
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile) r.across[tile][e] = to_float(theirs[z.k_first + head * D + 16 * tile + i]);
  }
}

// grid (vdim / (16 VT), heads, requests * segments), one wave a workgroup, which owns VT tiles of 16 value columns:
// Q, K and the scores are loaded, activated and computed once for all of them.  A request's tokens are cut into
// segments of `segment` tokens (a multiple of 16) that are walked side by side: the first starts from the request's
// state, the others from nothing, and each leaves the state it ends with in `carry` [requests * segments, heads, D,
// vdim]; the two kernels below then hand the states on and add what a segment's tokens read of the state they start
// from.  With one segment (`carry` null) the state is read and written here and nothing follows.
template <typename T, bool SILU, int VT>
__global__ __launch_bounds__(64) void decay_attention_runs_kernel(const T* __restrict__ x, DecaySizes z,
                                                                  const float* __restrict__ decays,
                                                                  const int* __restrict__ query_start,
                                                                  const int* __restrict__ state_slots, float* __restrict__ state,
                                                                  float* __restrict__ out, int segment, int segments,
                                                                  float* __restrict__ carry) {
  __shared__ float power[RUN + 1];
  const int v0 = blockIdx.x * 16 * VT, head = blockIdx.y, request = blockIdx.z / segments, part = blockIdx.z % segments;
  const int lane = threadIdx.x, i = lane & 15, g = lane >> 4;
  const int begin = query_start[request] + part * segment, end = min(query_start[request + 1], begin + segment);
  if (begin >= end) return;  // a request that only pads a captured step, or one with fewer segments
  if (lane <= RUN) power[lane] = (float)whole_power((double)decays[head], lane);
  __syncthreads();
  // S[d][v] of this wave's columns: lane (i, g) holds rows 16 tile + 4 g + e of columns v0 + 16 j + i
  float* s_at = state + (((size_t)state_slots[request] * z.heads + head) * D + 4 * g) * z.vdim + v0 + i;
  f32x4 S[VT][D_TILES];
#pragma unroll
  for (int j = 0; j < VT; ++j)
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) S[j][tile][e] = part == 0 ? s_at[(size_t)(16 * tile + e) * z.vdim + 16 * j] : 0.f;
  const int out_width = z.heads * z.vdim;

  RunOperands<VT> next;
  load_run(next, x, z, head, v0, begin, min(RUN, end - begin), i, g);
  for (int t0 = begin; t0 < end; t0 += RUN) {
    const int n = min(RUN, end - t0);
    RunOperands<VT> now = next;
    // The next run's operands are on their way while this run is computed.  (No branch around the loads: a wave waits at
    // a branch's end for what was asked for inside it.  After the last run, that run is asked for again and not used.)
    const int ahead = t0 + RUN < end ? t0 + RUN : t0;
    load_run(next, x, z, head, v0, ahead, min(RUN, end - ahead), i, g);
    const bool live = i < n;  // (a token beyond the run counts as zeros)
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        now.q[tile][e] = live ? activated_fast<SILU>(now.q[tile][e]) : 0.f;
        now.k[tile][e] = live ? activated_fast<SILU>(now.k[tile][e]) : 0.f;
      }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int s = 4 * g + e;
#pragma unroll
      for (int j = 0; j < VT; ++j) now.v[j][e] = s < n ? activated_fast<SILU>(now.v[j][e]) : 0.f;
      const float fade = s < n ? power[n - 1 - s] : 0.f;
#pragma unroll
      for (int tile = 0; tile < D_TILES; ++tile) now.across[tile][e] = s < n ? activated_fast<SILU>(now.across[tile][e]) * fade : 0.f;
    }
    // P^T[s][t] = k_s . q_t, faded by decay^(t - s) where s <= t
    f32x4 p = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) p = __builtin_amdgcn_mfma_f32_16x16x4f32(now.k[tile][e], now.q[tile][e], p, 0, 0, 0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int s = 4 * g + e;
      p[e] = s <= i ? p[e] * power[i - s] : 0.f;
    }
    const float carried = power[i + 1];
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) now.q[tile][e] *= carried;
    const float whole = power[n];
#pragma unroll
    for (int j = 0; j < VT; ++j) {
      // O[t][v] = sum_s P[t][s] V[s][v] + sum_d decay^(t+1) Q[t][d] S[d][v]
      f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int e = 0; e < 4; ++e) o = __builtin_amdgcn_mfma_f32_16x16x4f32(p[e], now.v[j][e], o, 0, 0, 0);
#pragma unroll
      for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
        for (int e = 0; e < 4; ++e) o = __builtin_amdgcn_mfma_f32_16x16x4f32(now.q[tile][e], S[j][tile][e], o, 0, 0, 0);
      // S = decay^n S + sum_s decay^(n-1-s) k_s v_s^T
#pragma unroll
      for (int tile = 0; tile < D_TILES; ++tile) {
#pragma unroll
        for (int e = 0; e < 4; ++e) S[j][tile][e] *= whole;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          S[j][tile] = __builtin_amdgcn_mfma_f32_16x16x4f32(now.across[tile][e], now.v[j][e], S[j][tile], 0, 0, 0);
      }
      // lane (i, g) holds O[t = 4 g + e][v0 + 16 j + i]
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (4 * g + e < n) out[(size_t)(t0 + 4 * g + e) * out_width + head * z.vdim + v0 + 16 * j + i] = o[e];
    }
  }
  float* left = carry ? carry + (((size_t)blockIdx.z * z.heads + head) * D + 4 * g) * z.vdim + v0 + i : s_at;
#pragma unroll
  for (int j = 0; j < VT; ++j)
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) left[(size_t)(16 * tile + e) * z.vdim + 16 * j] = S[j][tile][e];
}

// The states handed on from segment to segment, one thread an element of S: what segment j left, F_j = decay^(its
// tokens) F_(j-1) + its own sum, goes to the request's state after the last segment; carry[j] becomes F_(j-1), the state
// segment j starts from.  grid (ceil(D * vdim / 256), heads, requests).
__global__ __launch_bounds__(256) void decay_carry_kernel(DecaySizes z, const float* __restrict__ decays,
                                                          const int* __restrict__ query_start,
                                                          const int* __restrict__ state_slots, float* __restrict__ state,
                                                          int segment, int segments, float* __restrict__ carry) {
  const int element = blockIdx.x * blockDim.x + threadIdx.x, head = blockIdx.y, request = blockIdx.z;
  const int count = query_start[request + 1] - query_start[request];
  if (element >= D * z.vdim || count <= 0) return;
  const int used = (count + segment - 1) / segment;
  const size_t per_segment = (size_t)z.heads * D * z.vdim, at = (size_t)head * D * z.vdim + element;
  float* mine = carry + (size_t)request * segments * per_segment + at;
  const double decay = (double)decays[head];
  const float full = (float)whole_power(decay, segment);
  float running = mine[0];
  for (int j = 1; j < used; ++j) {
    const int tokens = min(segment, count - j * segment);
    const float own = mine[(size_t)j * per_segment];
    mine[(size_t)j * per_segment] = running;
    running = (tokens == segment ? full : (float)whole_power(decay, tokens)) * running + own;
  }
  state[(size_t)state_slots[request] * per_segment + at] = running;
}

// What the tokens of segments after the first read of the state their segment starts from:
// out[t][v] += decay^(t - segment's first + 1) sum_d Q[t][d] S_in[d][v].  grid as the kernel of runs.
template <typename T, bool SILU>
__global__ __launch_bounds__(64) void decay_attention_carried_kernel(const T* __restrict__ x, DecaySizes z,
                                                                     const float* __restrict__ decays,
                                                                     const int* __restrict__ query_start, float* __restrict__ out,
                                                                     int segment, int segments, const float* __restrict__ carry) {
  __shared__ float power[RUN + 1];
  const int v0 = blockIdx.x * 16, head = blockIdx.y, request = blockIdx.z / segments, part = blockIdx.z % segments;
  const int lane = threadIdx.x, i = lane & 15, g = lane >> 4;
  const int begin = query_start[request] + part * segment, end = min(query_start[request + 1], begin + segment);
  if (part == 0 || begin >= end) return;
  const double decay = (double)decays[head];
  if (lane <= RUN) power[lane] = (float)whole_power(decay, lane);
  __syncthreads();
  const float* s_at = carry + (((size_t)blockIdx.z * z.heads + head) * D + 4 * g) * z.vdim + v0 + i;
  f32x4 S[D_TILES];
#pragma unroll
  for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
    for (int e = 0; e < 4; ++e) S[tile][e] = s_at[(size_t)(16 * tile + e) * z.vdim];
  const int out_width = z.heads * z.vdim;
  const double run_decay = whole_power(decay, RUN);
  double before = 1.0;  // decay^(tokens of the segment before this run)
  for (int t0 = begin; t0 < end; t0 += RUN, before *= run_decay) {
    const int n = min(RUN, end - t0);
    const T* mine = x + (size_t)(t0 + min(i, n - 1)) * z.x_width + head * D + 4 * g + z.q_first;
    f32x4 q[D_TILES];
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile) q[tile] = load_four(mine + 16 * tile);
    float old[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) old[e] = out[(size_t)(t0 + min(4 * g + e, n - 1)) * out_width + head * z.vdim + v0 + i];
    const float carried = i < n ? (float)before * power[i + 1] : 0.f;
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int tile = 0; tile < D_TILES; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o = __builtin_amdgcn_mfma_f32_16x16x4f32(activated_fast<SILU>(q[tile][e]) * carried, S[tile][e], o, 0, 0, 0);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (4 * g + e < n) out[(size_t)(t0 + 4 * g + e) * out_width + head * z.vdim + v0 + i] = old[e] + o[e];
  }
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
// `longest` is the most tokens a request of the step brings (or may bring, in a step that is replayed).  The kernel
// of runs cuts a request's tokens into `segments` segments of `segment` tokens (a multiple of 16; segment * segments >=
// longest) that are walked side by side; with more than one, `carry` is float32 [requests * segments, heads, HEAD_DIM,
// vdim] of scratch.
extern "C" int llmserve_decay_attention(const void* x, int is_float, int tokens, int x_width, int q_first, int k_first, int v_first,
                                        int heads, int vdim, int activation, const float* decays, const int* query_start,
                                        const int* state_slots, int requests, int longest, float* state, float* out,
                                        int segment, int segments, float* carry, hipStream_t stream) {
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
  if (longest > 3 && vdim % 16 == 0 && x_width % 4 == 0 && q_first % 4 == 0 && k_first % 4 == 0) {
    if (segments < 1 || segment < RUN || segment % RUN || (segments > 1 && !carry) || (long)requests * segments > 65535 ||
        (long)segment * segments < longest)
      return ERR_BAD_ARGUMENT;
    float* kept = segments > 1 ? carry : nullptr;
    // How many tiles of 16 value columns a wave owns: what it loads and activates of Q and K serves them all, so as many
    // (1, 2 or 4; one where S's rows alone fill the registers) as still leave a wave for three SIMDs in four.
    const long tiles = (long)(vdim / 16) * heads * requests * segments;
    const int most = D <= 128 ? 4 : 1;
    int owned = 1;
    while (owned < most && vdim % (32 * owned) == 0 && tiles / (2 * owned) >= 768) owned *= 2;
    dim3 grid(vdim / (16 * owned), heads, requests * segments);
#define LAUNCH_RUNS(KERNEL, ...)                                                                                                 \
  do {                                                                                                                          \
    if (is_float && activation) hipLaunchKernelGGL((KERNEL<float, true>), grid, dim3(64), 0, stream, (const float*)x, __VA_ARGS__);   \
    else if (is_float) hipLaunchKernelGGL((KERNEL<float, false>), grid, dim3(64), 0, stream, (const float*)x, __VA_ARGS__);         \
    else if (activation) hipLaunchKernelGGL((KERNEL<bf16_t, true>), grid, dim3(64), 0, stream, (const bf16_t*)x, __VA_ARGS__);      \
    else hipLaunchKernelGGL((KERNEL<bf16_t, false>), grid, dim3(64), 0, stream, (const bf16_t*)x, __VA_ARGS__);                     \
  } while (0)
#define LAUNCH_OWNED(VT)                                                                                                         \
  do {                                                                                                                          \
    if (is_float && activation) hipLaunchKernelGGL((decay_attention_runs_kernel<float, true, VT>), grid, dim3(64), 0, stream, (const float*)x, z, decays, query_start, state_slots, state, out, segment, segments, kept);   \
    else if (is_float) hipLaunchKernelGGL((decay_attention_runs_kernel<float, false, VT>), grid, dim3(64), 0, stream, (const float*)x, z, decays, query_start, state_slots, state, out, segment, segments, kept);         \
    else if (activation) hipLaunchKernelGGL((decay_attention_runs_kernel<bf16_t, true, VT>), grid, dim3(64), 0, stream, (const bf16_t*)x, z, decays, query_start, state_slots, state, out, segment, segments, kept);      \
    else hipLaunchKernelGGL((decay_attention_runs_kernel<bf16_t, false, VT>), grid, dim3(64), 0, stream, (const bf16_t*)x, z, decays, query_start, state_slots, state, out, segment, segments, kept);                     \
  } while (0)
    if (owned == 4) LAUNCH_OWNED(most >= 4 ? 4 : 1);
    else if (owned == 2) LAUNCH_OWNED(most >= 2 ? 2 : 1);
    else LAUNCH_OWNED(1);
#undef LAUNCH_OWNED
    grid = dim3(vdim / 16, heads, requests * segments);
    if (segments > 1) {
      hipLaunchKernelGGL(decay_carry_kernel, dim3((D * vdim + 255) / 256, heads, requests), dim3(256), 0, stream, z, decays,
                         query_start, state_slots, state, segment, segments, carry);
      LAUNCH_RUNS(decay_attention_carried_kernel, z, decays, query_start, out, segment, segments, (const float*)carry);
    }
#undef LAUNCH_RUNS
    return LAUNCH_STATUS();
  }
#endif
  LAUNCH_DECAY(decay_attention_tokens_kernel, dim3((vdim + 63) / 64, heads, requests), TOKEN_WAVES * 64);
#undef LAUNCH_DECAY
  return LAUNCH_STATUS();
}
