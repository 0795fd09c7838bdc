// The gated delta rule and what stands around it: short causal convolutions over a request's tokens with their
// last inputs kept per request, the recurrence over a matrix state per head, and the gated norm of its read-out.
// Everything that enters the recurrence is float32; projections come in bfloat16 or float32.
#include "common.h"

// ---------------------------------------------------------------------------- short causal convolution + silu
// Request b brings the tokens [start[b], start[b + 1]) of the step.  For its token number i (from 0) and channel c
//   y[i, c] = silu(sum_j taps[c, j] * in(i - (width - 1) + j, c) (+ bias[c]))      (`plain`: without the silu),
// where in(n, c) is the step's own input for n >= 0 and, for n < 0, the request's kept input number width - 1 + n
// (window[slot, width - 1 + n, c]: the last width - 1 inputs of earlier steps, zeros at a request's start).
// One thread per (token, channel); the window is read here and written by the kernel below.
#define MAX_TAPS 16
template <typename T>
__global__ void causal_conv_kernel(const T* __restrict__ x, int x_stride, int channels, const float* __restrict__ taps,
                                   int width, const int* __restrict__ token_request, const int* __restrict__ start,
                                   const int* __restrict__ slots, const float* __restrict__ window, T* __restrict__ out,
                                   const float* __restrict__ bias, int plain) {
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
  if (bias) sum += bias[c];
  out[(size_t)t * channels + c] = from_float<T>(plain ? sum : sum / (1.f + expf(-sum)));
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
                                    float* window, void* out, const float* bias, int plain, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (width < 1 || width > MAX_TAPS || channels < 1 || channels > x_stride || (width > 1 && !window)) return ERR_BAD_ARGUMENT;
  const int threads = channels <= 64 ? 64 : channels <= 128 ? 128 : 256;
  const dim3 grid(tokens, (channels + threads - 1) / threads);
  if (is_float)
    hipLaunchKernelGGL(causal_conv_kernel<float>, grid, dim3(threads), 0, stream, (const float*)x, x_stride, channels, taps, width,
                       token_request, start, slots, (const float*)window, (float*)out, bias, plain);
  else
    hipLaunchKernelGGL(causal_conv_kernel<bf16_t>, grid, dim3(threads), 0, stream, (const bf16_t*)x, x_stride, channels, taps,
                       width, token_request, start, slots, (const float*)window, (bf16_t*)out, bias, plain);
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
//
// Two kernels.  The first is parallel over tokens: it makes q and k unit vectors and the decays and betas, all in
// float32, and leaves them as the second wants to read them.  The second walks a request's tokens in order.  Column j of
// S (the state of value dimension j) never meets another column: sixteen neighbouring lanes share a column, each keeping
// ROWS of its rows in registers for all the tokens of the request's step, and the two sums over a column's rows end with
// four exchanges between those lanes; a workgroup of four waves owns sixteen columns of one (request, head).  The tokens
// are walked in runs of RUN: while a run is worked through out of LDS and registers, the next run's k, q, decays, betas
// and v are on their way from memory into registers (a token by itself would wait for memory every time).  The state is
// kept as S^T (state[slot, h] is [vdim, dim]: a lane's rows lie side by side) and goes back after the step's last token.
#define RUN 16
#define LANES_A_COLUMN 16

// The sum over the sixteen lanes of a row (lanes 16 i .. 16 i + 15), left in every one of them: the lanes are moved by the
// data-parallel primitives of the vector unit (pairs, pairs of pairs, then the row turned by four and by eight lanes), a
// few cycles each, where an exchange through the LDS crossbar takes ten times as long; the recurrence waits for two such
// sums a token.
__device__ __forceinline__ float moved(float v, int how) {
  switch (how) {  // (constants: the primitive takes its pattern as an immediate)
    case 0: return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm [1, 0, 3, 2]
    case 1: return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm [2, 3, 0, 1]
    case 2: return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xF, 0xF, true));  // row_ror 4
    default: return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, true)); // row_ror 8
  }
}
__device__ __forceinline__ float row_sum(float v) {
  v += moved(v, 0);
  v += moved(v, 1);
  v += moved(v, 2);
  v += moved(v, 3);
  return v;
}
#define COLUMNS 16  // a workgroup's: 256 threads / LANES_A_COLUMN

__host__ __device__ constexpr int delta_rows(int dim) { return 4 * ((dim + 63) / 64); }      // rows a lane keeps
__host__ __device__ constexpr int delta_line(int rows) { return LANES_A_COLUMN * (rows + 4); }  // a vector in LDS: 4 floats between the lanes' shares (banks)

extern "C" int llmserve_delta_line(int dim) { return delta_line(delta_rows(dim)); }

// The unit vectors of one (token, query/key head) as the recurrence reads them, written by one wave: element i of a
// vector lies at (i / rows) * (rows + 4) + i % rows of its `line` floats, zeros elsewhere.  q(i), k(i) give the elements.
// With a decay per key channel (`steps`: what the softplus takes, before its bias, [heads * dim] a token) a head has a third
// vector, exp(-exp(rate_h) softplus(step + bias)), and the place is the value head's: [k | q | g].
template <typename Q, typename K>
__device__ __forceinline__ void write_unit_vectors(Q q_of, K k_of, int dim, int rows, int line, int lane, float* dst, const float* steps,
                                                   const float* step_bias, float rate) {
  const float q_scale = rsqrtf((float)dim);
  float q[4], k[4], q_squares = 0.f, k_squares = 0.f;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int i = p * WAVE + lane;
    q[p] = i < dim ? q_of(i) : 0.f;
    k[p] = i < dim ? k_of(i) : 0.f;
    q_squares += q[p] * q[p];
    k_squares += k[p] * k[p];
  }
  const float q_unit = q_scale / sqrtf(wave_sum(q_squares) + 1e-6f), k_unit = 1.f / sqrtf(wave_sum(k_squares) + 1e-6f);
  const int vectors = steps ? 3 : 2;
  for (int i = lane; i < vectors * line; i += WAVE) dst[i] = i < 2 * line ? 0.f : 1.f;  // (the gaps and what lies beyond dim; this wave alone writes here)
  __builtin_amdgcn_s_waitcnt(0);
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int i = p * WAVE + lane;
    if (i < dim) {
      const int where = (i / rows) * (rows + 4) + i % rows;
      dst[where] = k[p] * k_unit;
      dst[line + where] = q[p] * q_unit;
      if (steps) {
        const float a_in = steps[i] + step_bias[i];
        const float softplus = a_in > 20.f ? a_in : log1pf(expf(a_in));
        dst[2 * line + where] = expf(-rate * softplus);
      }
    }
  }
}

// unit[t, kv head] = [k | q], each `line` floats: element i of the vector at (i / rows) * (rows + 4) + i % rows, zeros elsewhere.
// gates[t, head] = (g, beta).  One workgroup a token, a wave a kv head in turn.
template <typename T>
__global__ __launch_bounds__(256) void delta_prepare_kernel(const T* __restrict__ mixed, const float* __restrict__ controls,
                                                            const float* __restrict__ rate, const float* __restrict__ step_bias,
                                                            int heads, int kv_heads, int dim, int vdim, int rows, int line,
                                                            float* __restrict__ unit, float* __restrict__ gates,
                                                            const float* __restrict__ steps, int steps_stride) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* row = mixed + (size_t)t * (2 * kv_heads * dim + heads * vdim);
  if (steps) {
    for (int head = wave; head < heads; head += 4) {
      const int kv_head = head / (heads / kv_heads);
      write_unit_vectors([&](int i) { return to_float(row[kv_head * dim + i]); }, [&](int i) { return to_float(row[(kv_heads + kv_head) * dim + i]); },
                         dim, rows, line, lane, unit + ((size_t)t * heads + head) * 3 * line, steps + (size_t)t * steps_stride + head * dim,
                         step_bias + head * dim, expf(rate[head]));
    }
  } else {
    for (int kv_head = wave; kv_head < kv_heads; kv_head += 4)
      write_unit_vectors([&](int i) { return to_float(row[kv_head * dim + i]); }, [&](int i) { return to_float(row[(kv_heads + kv_head) * dim + i]); },
                         dim, rows, line, lane, unit + ((size_t)t * kv_heads + kv_head) * 2 * line, nullptr, nullptr, 0.f);
  }
  for (int head = threadIdx.x; head < heads; head += blockDim.x) {
    const int controls_stride = steps ? heads : 2 * heads;
    const float b_in = controls[(size_t)t * controls_stride + head];
    float decay = 1.f;
    if (!steps) {
      const float a_in = controls[(size_t)t * 2 * heads + heads + head] + step_bias[head];
      const float softplus = a_in > 20.f ? a_in : log1pf(expf(a_in));
      decay = expf(-expf(rate[head]) * softplus);
    }
    gates[((size_t)t * heads + head) * 2] = decay;
    gates[((size_t)t * heads + head) * 2 + 1] = 1.f / (1.f + expf(-b_in));
  }
}

// One channel's convolution at token number i0 of its request, silu applied.  WIDTH > 0: the taps are known when the
// kernel is compiled and all their loads are asked for together; WIDTH 0: any number of taps, one after the other.
template <typename T, int WIDTH>
__device__ __forceinline__ float convolved_channel(const T* __restrict__ x, int x_stride, int channels, const float* __restrict__ taps,
                                                   int width, const float* __restrict__ kept, int t, int i0, int c) {
  float sum = 0.f;
  if (WIDTH > 0) {
    float v[WIDTH > 0 ? WIDTH : 1], w[WIDTH > 0 ? WIDTH : 1];
#pragma unroll
    for (int j = 0; j < WIDTH; ++j) {
      const int n = i0 - (WIDTH - 1) + j;
      // (both addresses are valid whichever is meant: no load stands in a branch)
      const float fresh = to_float(x[(size_t)(t - i0 + max(n, 0)) * x_stride + c]);
      const float old = WIDTH > 1 ? kept[(size_t)min(WIDTH - 1 + n, WIDTH - 2) * channels + c] : 0.f;
      v[j] = n >= 0 ? fresh : old;
      w[j] = taps[(size_t)c * WIDTH + j];
    }
#pragma unroll
    for (int j = 0; j < WIDTH; ++j) sum += w[j] * v[j];
  } else {
    for (int j = 0; j < width; ++j) {
      const int n = i0 - (width - 1) + j;
      const float v = n >= 0 ? to_float(x[(size_t)(t - i0 + n) * x_stride + c]) : kept[(size_t)(width - 1 + n) * channels + c];
      sum += taps[(size_t)c * width + j] * v;
    }
  }
  return sum / (1.f + expf(-sum));
}

// The same with the convolutions in front: the token's row of x is [q | k | v | ...] before the convolutions, `channels`
// of them; the workgroup convolves them (as causal_conv_kernel does), keeps the results in LDS as float32, and goes on
// as above; the convolved v goes to values[t] (float32 [heads * vdim]).  The window is read here and written by the
// recurrence kernel, which runs behind this one.
template <typename T, int WIDTH>
__global__ __launch_bounds__(1024) void delta_prepare_conv_kernel(const T* __restrict__ x, int x_stride, int channels,
                                                                 const float* __restrict__ taps, int width,
                                                                 const int* __restrict__ token_request, const int* __restrict__ start,
                                                                 const int* __restrict__ slots, const float* __restrict__ window,
                                                                 const float* __restrict__ controls, const float* __restrict__ rate,
                                                                 const float* __restrict__ step_bias, int heads, int kv_heads, int dim,
                                                                 int vdim, int rows, int line, float* __restrict__ unit,
                                                                 float* __restrict__ gates, float* __restrict__ values,
                                                                 const float* __restrict__ steps, int steps_stride) {
  extern __shared__ float convolved[];  // [channels]
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int b = token_request[t], i0 = t - start[b];
  const float* kept = window ? window + (size_t)slots[b] * (width - 1) * channels : nullptr;
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    const float y = convolved_channel<T, WIDTH>(x, x_stride, channels, taps, width, kept, t, i0, c);
    convolved[c] = y;
    if (c >= 2 * kv_heads * dim) values[(size_t)t * heads * vdim + c - 2 * kv_heads * dim] = y;
  }
  __syncthreads();
  if (steps) {
    for (int head = wave; head < heads; head += blockDim.x / WAVE) {
      const int kv_head = head / (heads / kv_heads);
      write_unit_vectors([&](int i) { return convolved[kv_head * dim + i]; }, [&](int i) { return convolved[(kv_heads + kv_head) * dim + i]; },
                         dim, rows, line, lane, unit + ((size_t)t * heads + head) * 3 * line, steps + (size_t)t * steps_stride + head * dim,
                         step_bias + head * dim, expf(rate[head]));
    }
  } else {
    for (int kv_head = wave; kv_head < kv_heads; kv_head += blockDim.x / WAVE)
      write_unit_vectors([&](int i) { return convolved[kv_head * dim + i]; }, [&](int i) { return convolved[(kv_heads + kv_head) * dim + i]; },
                         dim, rows, line, lane, unit + ((size_t)t * kv_heads + kv_head) * 2 * line, nullptr, nullptr, 0.f);
  }
  for (int head = threadIdx.x; head < heads; head += blockDim.x) {
    const int controls_stride = steps ? heads : 2 * heads;
    const float b_in = controls[(size_t)t * controls_stride + head];
    float decay = 1.f;
    if (!steps) {
      const float a_in = controls[(size_t)t * 2 * heads + heads + head] + step_bias[head];
      const float softplus = a_in > 20.f ? a_in : log1pf(expf(a_in));
      decay = expf(-expf(rate[head]) * softplus);
    }
    gates[((size_t)t * heads + head) * 2] = decay;
    gates[((size_t)t * heads + head) * 2 + 1] = 1.f / (1.f + expf(-b_in));
  }
}

// VECS 2: a decay a head, the run's vectors are [k | q] of the query/key head.  VECS 3: a decay a key channel, the vectors
// are [k | q | g] of the value head, and row r of S is scaled by g[r].
template <typename T, int ROWS, int TOKENS, int VECS>  // 16 * ROWS >= dim; TOKENS: a run's tokens (RUN, or 2 where every request brings one or two)
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(const T* __restrict__ mixed, const float* __restrict__ values,
                                                               const float* __restrict__ unit, const float* __restrict__ gates,
                                                               int heads, int kv_heads, int dim, int vdim,
                                                               const int* __restrict__ start, const int* __restrict__ slots,
                                                               float* __restrict__ state, float* __restrict__ out,
                                                               const T* __restrict__ x, int x_stride, int channels, int width,
                                                               float* __restrict__ window) {
  constexpr int LINE = delta_line(ROWS), QUADS = TOKENS * VECS * LINE / 4, MINE = (QUADS + 255) / 256;  // float4 of a run, and a thread's share
  __shared__ __attribute__((aligned(16))) float vectors[TOKENS][VECS][LINE];
  __shared__ float decay_beta[TOKENS][2];
  const int b = blockIdx.x, head = blockIdx.y, thread = threadIdx.x;
  const int column = blockIdx.z * COLUMNS + thread / LANES_A_COLUMN, share = thread % LANES_A_COLUMN;
  const bool owns = column < vdim;
  const int first = start[b], last = start[b + 1];
  if (last <= first) return;
  if (window) {
    // With the convolutions in the kernel before this one (`values` given): the request's kept inputs move on, as
    // conv_window_kernel does it, the channels dealt out to the request's workgroups; every thread reads what it needs
    // of a channel before it writes.
    float* kept = window + (size_t)slots[b] * (width - 1) * channels;
    const int count = last - first;
    for (int c = (head * gridDim.z + blockIdx.z) * 256 + thread; c < channels; c += gridDim.y * gridDim.z * 256) {
      float next[MAX_TAPS];
#pragma unroll
      for (int i = 0; i < MAX_TAPS; ++i) {
        if (i < width - 1) {
          const int n = count - (width - 1) + i;
          next[i] = n >= 0 ? to_float(x[(size_t)(first + n) * x_stride + c]) : kept[(size_t)(i + count) * channels + c];
        }
      }
#pragma unroll
      for (int i = 0; i < MAX_TAPS; ++i)
        if (i < width - 1) kept[(size_t)i * channels + c] = next[i];
    }
  }
  const int kv_head = head / (heads / kv_heads);
  const int row_width = 2 * kv_heads * dim + heads * vdim;
  float* mine = state + (((size_t)slots[b] * heads + head) * vdim + column) * dim + share * ROWS;
  float S[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) S[r] = (owns && share * ROWS + r < dim) ? mine[r] : 0.f;

  float4 coming[MINE];
  float v_coming[TOKENS], gate_coming = 0.f;
  // Asks memory for the run that begins at t0: token c of it is quad / (2 LINE / 4) of the run's quads.  The loads stand
  // in no branch (one would make the wave wait for them at its end): a token beyond the request's last is read from the
  // last one's place, and `keep` puts zeros for its k and q, a decay of one and a beta of zero instead: walking it changes
  // nothing, so the walk below has no branches either, and one token's vectors are read before the sums of the token before.
  auto ask = [&](int t0) {
#pragma unroll
    for (int j = 0; j < MINE; ++j) {
      const int quad = min(thread + j * 256, QUADS - 1);
      const int c = quad / (VECS * LINE / 4), inside = quad % (VECS * LINE / 4);
      coming[j] = ((const float4*)(unit + ((size_t)min(t0 + c, last - 1) * (VECS == 3 ? heads : kv_heads) + (VECS == 3 ? head : kv_head)) * VECS * LINE))[inside];
    }
    const int my_column = min(column, vdim - 1);
#pragma unroll
    for (int c = 0; c < TOKENS; ++c)
      v_coming[c] = values ? values[(size_t)min(t0 + c, last - 1) * heads * vdim + head * vdim + my_column]
                           : to_float(mixed[(size_t)min(t0 + c, last - 1) * row_width + 2 * kv_heads * dim + head * vdim + my_column]);
    gate_coming = gates[((size_t)min(t0 + (thread / 2) % TOKENS, last - 1) * heads + head) * 2 + thread % 2];
  };
  auto keep = [&](int t0) {
#pragma unroll
    for (int j = 0; j < MINE; ++j) {
      const int quad = thread + j * 256;
      const int c = quad / (VECS * LINE / 4);
      const float absent = quad % (VECS * LINE / 4) >= 2 * LINE / 4 ? 1.f : 0.f;  // (a token beyond the end: k = q = 0, and decays of one)
      if (quad < QUADS) ((float4*)&vectors[0][0][0])[quad] = t0 + c < last ? coming[j] : make_float4(absent, absent, absent, absent);
    }
    if (thread < 2 * TOKENS) decay_beta[thread / 2][thread % 2] = t0 + thread / 2 < last ? gate_coming : (thread % 2 ? 0.f : 1.f);
  };

  ask(first);
  keep(first);
  float v[TOKENS];
#pragma unroll
  for (int c = 0; c < TOKENS; ++c) v[c] = v_coming[c];
  __syncthreads();
  for (int t0 = first; t0 < last; t0 += TOKENS) {
    const bool more = t0 + TOKENS < last;
    ask(t0 + TOKENS);  // (beyond the last run: the last token again, dropped)
    float4 key[ROWS / 4], query[ROWS / 4], next_key[ROWS / 4], next_query[ROWS / 4], fade[ROWS / 4], next_fade[ROWS / 4];
    float g = decay_beta[0][0], beta = decay_beta[0][1], next_g = 1.f, next_beta = 0.f;
#pragma unroll
    for (int r = 0; r < ROWS / 4; ++r) {
      key[r] = ((const float4*)&vectors[0][0][share * (ROWS + 4)])[r];
      query[r] = ((const float4*)&vectors[0][1][share * (ROWS + 4)])[r];
      if (VECS == 3) fade[r] = ((const float4*)&vectors[0][VECS - 1][share * (ROWS + 4)])[r];
    }
#pragma unroll
    for (int c = 0; c < TOKENS; ++c) {
      if (c + 1 < TOKENS) {
        next_g = decay_beta[c + 1][0];
        next_beta = decay_beta[c + 1][1];
#pragma unroll
        for (int r = 0; r < ROWS / 4; ++r) {
          next_key[r] = ((const float4*)&vectors[c + 1][0][share * (ROWS + 4)])[r];
          next_query[r] = ((const float4*)&vectors[c + 1][1][share * (ROWS + 4)])[r];
          if (VECS == 3) next_fade[r] = ((const float4*)&vectors[c + 1][VECS - 1][share * (ROWS + 4)])[r];
        }
      }
      float seen = 0.f, seen_too = 0.f;  // (g S)^T k over this lane's rows, in two chains
#pragma unroll
      for (int r = 0; r < ROWS; r += 4) {
        const float4 kk = key[r / 4];
        if (VECS == 3) {
          const float4 gg = fade[r / 4];
          S[r] *= gg.x; S[r + 1] *= gg.y; S[r + 2] *= gg.z; S[r + 3] *= gg.w;
        } else {
          S[r] *= g; S[r + 1] *= g; S[r + 2] *= g; S[r + 3] *= g;
        }
        seen += S[r] * kk.x; seen_too += S[r + 1] * kk.y; seen += S[r + 2] * kk.z; seen_too += S[r + 3] * kk.w;
      }
      seen = row_sum(seen + seen_too);
      const float u = beta * (v[c] - seen);
      float read = 0.f, read_too = 0.f;
#pragma unroll
      for (int r = 0; r < ROWS; r += 4) {
        const float4 kk = key[r / 4], qq = query[r / 4];
        S[r] += kk.x * u; S[r + 1] += kk.y * u; S[r + 2] += kk.z * u; S[r + 3] += kk.w * u;
        read += S[r] * qq.x; read_too += S[r + 1] * qq.y; read += S[r + 2] * qq.z; read_too += S[r + 3] * qq.w;
      }
      read = row_sum(read + read_too);
      if (owns && share == 0 && t0 + c < last) out[(size_t)(t0 + c) * heads * vdim + head * vdim + column] = read;
      g = next_g;
      beta = next_beta;
#pragma unroll
      for (int r = 0; r < ROWS / 4; ++r) {
        key[r] = next_key[r];
        query[r] = next_query[r];
        if (VECS == 3) fade[r] = next_fade[r];
      }
    }
    __syncthreads();  // everybody has read this run
    if (more) {
      keep(t0 + TOKENS);
#pragma unroll
      for (int c = 0; c < TOKENS; ++c) v[c] = v_coming[c];
    }
    __syncthreads();
  }
  if (owns) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
      if (share * ROWS + r < dim) mine[r] = S[r];
  }
}

// `unit` has room for tokens * kv_heads * 2 * llmserve_delta_line(dim) floats (with a decay per key channel: tokens * heads * 3
// of them), `gates` for tokens * heads * 2.  `steps` (null: a decay a head, from `controls`' second half) is what the
// channels' softplus takes before its bias, float32 [tokens, steps_stride], the first heads * dim columns of it.
// `longest`: the most tokens a request brings; one or two (decoding) are walked in runs of two.
template <typename T>
static int launch_rule(const T* mixed, const float* values, const float* unit, const float* gates, int heads, int kv_heads, int dim,
                       int vdim, const int* start, const int* slots, int requests, int longest, float* state, float* out, const T* x,
                       int x_stride, int channels, int width, float* window, int by_channel, hipStream_t stream) {
  const dim3 grid(requests, heads, (vdim + COLUMNS - 1) / COLUMNS);
  const int rows = delta_rows(dim);
#define LAUNCH_RULE_OF(ROWS, TOKENS, VECS)                                                                                         \
  hipLaunchKernelGGL((gated_delta_rule_kernel<T, ROWS, TOKENS, VECS>), grid, dim3(256), 0, stream, mixed, values, unit, gates, heads, \
                     kv_heads, dim, vdim, start, slots, state, out, x, x_stride, channels, width, window)
#define LAUNCH_RULE(ROWS)                                                                                                         \
  do {                                                                                                                            \
    if (by_channel) {                                                                                                             \
      if (longest <= 2) LAUNCH_RULE_OF(ROWS, 2, 3); else LAUNCH_RULE_OF(ROWS, RUN, 3);                                            \
    } else {                                                                                                                      \
      if (longest <= 2) LAUNCH_RULE_OF(ROWS, 2, 2); else LAUNCH_RULE_OF(ROWS, RUN, 2);                                            \
    }                                                                                                                             \
  } while (0)
  if (rows == 4) LAUNCH_RULE(4); else if (rows == 8) LAUNCH_RULE(8); else if (rows == 12) LAUNCH_RULE(12); else LAUNCH_RULE(16);
#undef LAUNCH_RULE
#undef LAUNCH_RULE_OF
  return LAUNCH_STATUS();
}

extern "C" int llmserve_gated_delta_rule(const void* mixed, int is_float, const float* controls, const float* rate,
                                         const float* step_bias, int heads, int kv_heads, int dim, int vdim, const int* start,
                                         const int* slots, int requests, int tokens, int longest, float* unit, float* gates,
                                         float* state, float* out, const float* steps, int steps_stride, hipStream_t stream) {
  if (requests <= 0 || tokens <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads || dim < 1 || dim > 256 || vdim < 1 || heads > 65535) return ERR_BAD_ARGUMENT;
  const int rows = delta_rows(dim), line = delta_line(rows);
  if (is_float) {
    hipLaunchKernelGGL(delta_prepare_kernel<float>, dim3(tokens), dim3(256), 0, stream, (const float*)mixed, controls, rate, step_bias,
                       heads, kv_heads, dim, vdim, rows, line, unit, gates, steps, steps_stride);
    return launch_rule<float>((const float*)mixed, nullptr, unit, gates, heads, kv_heads, dim, vdim, start, slots, requests, longest,
                              state, out, nullptr, 0, 0, 0, nullptr, steps != nullptr, stream);
  }
  hipLaunchKernelGGL(delta_prepare_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream, (const bf16_t*)mixed, controls, rate,
                     step_bias, heads, kv_heads, dim, vdim, rows, line, unit, gates, steps, steps_stride);
  return launch_rule<bf16_t>((const bf16_t*)mixed, nullptr, unit, gates, heads, kv_heads, dim, vdim, start, slots, requests, longest,
                             state, out, nullptr, 0, 0, 0, nullptr, steps != nullptr, stream);
}

// Convolutions, unit vectors, gates and the recurrence in two kernels: x [tokens, x_stride] holds [q | k | v] before the
// convolutions in its first `channels` columns; `values` has room for tokens * heads * vdim floats.
extern "C" int llmserve_conv_gated_delta_rule(const void* x, int is_float, int x_stride, int channels, const float* taps, int width,
                                              const int* token_request, float* window, const float* controls, const float* rate,
                                              const float* step_bias, int heads, int kv_heads, int dim, int vdim, const int* start,
                                              const int* slots, int requests, int tokens, int longest, float* unit, float* gates,
                                              float* values, float* state, float* out, const float* steps, int steps_stride,
                                              hipStream_t stream) {
  if (requests <= 0 || tokens <= 0) return 0;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads || dim < 1 || dim > 256 || vdim < 1 || heads > 65535) return ERR_BAD_ARGUMENT;
  if (width < 1 || width > MAX_TAPS || channels != 2 * kv_heads * dim + heads * vdim || channels > x_stride || channels > 12288 ||
      (width > 1 && !window))
    return ERR_BAD_ARGUMENT;
  const int rows = delta_rows(dim), line = delta_line(rows);
  const size_t lds = (size_t)channels * sizeof(float);
  const int threads = channels > 512 ? 1024 : 256;
#define LAUNCH_PREPARE(TYPE, WIDTH)                                                                                                  \
  hipLaunchKernelGGL((delta_prepare_conv_kernel<TYPE, WIDTH>), dim3(tokens), dim3(threads), lds, stream, (const TYPE*)x, x_stride,    \
                     channels, taps, width, token_request, start, slots, (const float*)window, controls, rate, step_bias, heads,     \
                     kv_heads, dim, vdim, rows, line, unit, gates, values, steps, steps_stride)
#define LAUNCH_PREPARE_BY_WIDTH(TYPE)                                                                                       \
  switch (width) {                                                                                                          \
    case 1: LAUNCH_PREPARE(TYPE, 1); break;                                                                                 \
    case 2: LAUNCH_PREPARE(TYPE, 2); break;                                                                                 \
    case 3: LAUNCH_PREPARE(TYPE, 3); break;                                                                                 \
    case 4: LAUNCH_PREPARE(TYPE, 4); break;                                                                                 \
    default: LAUNCH_PREPARE(TYPE, 0); break;                                                                                \
  }
  if (is_float) {
    LAUNCH_PREPARE_BY_WIDTH(float)
    return launch_rule<float>(nullptr, values, unit, gates, heads, kv_heads, dim, vdim, start, slots, requests, longest, state, out,
                              (const float*)x, x_stride, channels, width, width > 1 ? window : nullptr, steps != nullptr, stream);
  }
  LAUNCH_PREPARE_BY_WIDTH(bf16_t)
#undef LAUNCH_PREPARE_BY_WIDTH
#undef LAUNCH_PREPARE
  return launch_rule<bf16_t>(nullptr, values, unit, gates, heads, kv_heads, dim, vdim, start, slots, requests, longest, state, out,
                             (const bf16_t*)x, x_stride, channels, width, width > 1 ? window : nullptr, steps != nullptr, stream);
}

// ---------------------------------------------------------------------------- gated norm of the read-out
// out[t, h, :] = read[t, h, :] * rsqrt(mean(read[t, h, :]^2) + eps) * weight * silu(gates[t, gate_first + h * vdim + :]),
// one wave per (token, head).
template <typename G, typename T>
__global__ __launch_bounds__(512) void gated_head_norm_kernel(const float* __restrict__ read, const G* __restrict__ gates,
                                                             int gate_stride, int gate_first, const void* __restrict__ weight,
                                                             int weight_is_float, float eps, int vdim, int squash,
                                                             T* __restrict__ out) {
  const size_t base = ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * vdim;
  const G* gate = gates + (size_t)blockIdx.x * gate_stride + gate_first + (size_t)blockIdx.y * vdim;
  float squares = 0.f;
  __shared__ float shared[17];
  for (int i = threadIdx.x; i < vdim; i += blockDim.x) squares += read[base + i] * read[base + i];
  const float scale = rsqrtf((blockDim.x == WAVE ? wave_sum(squares) : block_sum(squares, shared)) / (float)vdim + eps);
  for (int i = threadIdx.x; i < vdim; i += blockDim.x) {
    const float z = to_float(gate[i]);
    const float gated = squash ? 1.f / (1.f + expf(-z)) : z / (1.f + expf(-z));  // sigmoid, or silu
    out[base + i] = from_float<T>(read[base + i] * scale * load_as_float(weight, weight_is_float, i) * gated);
  }
}

// The gates may be float32 where the result is bfloat16 (gates that a product left in float32).
extern "C" int llmserve_gated_head_norm(const float* read, const void* gates, int is_float, int gate_stride, int gate_first,
                                        const void* weight, int weight_is_float, float eps, int tokens, int heads, int vdim,
                                        int squash, int out_is_float, void* out, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads < 1 || heads > 65535 || vdim < 1 || gate_first + heads * vdim > gate_stride || (out_is_float && !is_float)) return ERR_BAD_ARGUMENT;
  const dim3 grid(tokens, heads);
  const int threads = vdim <= 256 ? WAVE : vdim <= 1024 ? 256 : 512;  // (a norm over all heads at once is one wide "head")
  if (is_float && out_is_float)
    hipLaunchKernelGGL((gated_head_norm_kernel<float, float>), grid, dim3(threads), 0, stream, read, (const float*)gates, gate_stride,
                       gate_first, weight, weight_is_float, eps, vdim, squash, (float*)out);
  else if (is_float)
    hipLaunchKernelGGL((gated_head_norm_kernel<float, bf16_t>), grid, dim3(threads), 0, stream, read, (const float*)gates, gate_stride,
                       gate_first, weight, weight_is_float, eps, vdim, squash, (bf16_t*)out);
  else
    hipLaunchKernelGGL((gated_head_norm_kernel<bf16_t, bf16_t>), grid, dim3(threads), 0, stream, read, (const bf16_t*)gates, gate_stride,
                       gate_first, weight, weight_is_float, eps, vdim, squash, (bf16_t*)out);
  return LAUNCH_STATUS();
}
