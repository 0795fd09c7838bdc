// A gated linear recurrence with a diagonal state.  For channel c of a request's token t:
//   r = sigmoid(gates[t, r_c] + bias[r_c]),  i = sigmoid(gates[t, i_c] + bias[i_c]),  log a = rates[c] * r,
//   S <- a S + sqrt(1 - a^2) * i * u[t, c],   out[t, c] = S * act(branch[t, c])
// where the gates' columns come in `blocks` parts of the channels, a part's r columns before its i columns.  Gates,
// decays and S are float32; u, the gates' products and the branch come in bfloat16 or float32.
//
// The state of a channel meets no other channel.  A workgroup owns 64 channels of one request; a long portion is cut
// into as many runs of tokens as the workgroup has rows of threads: every row first walks its run from an empty state and
// notes the product of its decays and what it ends with, then takes the state that the runs before it leave
// (S_end = A S_in + B, run after run) and walks its run again for the results.  The last row leaves the request's state.
#include "common.h"

#define CHANNELS 64
#define MAX_RUNS 16

template <typename T>
__global__ __launch_bounds__(CHANNELS * MAX_RUNS) void gated_recurrence_kernel(
    const T* __restrict__ u, const T* __restrict__ gates, const float* __restrict__ bias, const float* __restrict__ rates,
    const T* __restrict__ branch, int branch_stride, int branch_first, int width, int part, const int* __restrict__ start,
    const int* __restrict__ slots, float* __restrict__ state, T* __restrict__ out) {
  __shared__ float decays[MAX_RUNS][CHANNELS], ends[MAX_RUNS][CHANNELS];
  const int b = blockIdx.x, c = blockIdx.y * CHANNELS + threadIdx.x, run = threadIdx.y, runs = blockDim.y;
  const int first = start[b], count = start[b + 1] - first;
  if (count <= 0) return;
  const bool owns = c < width;
  const int mine = owns ? c : width - 1;  // (a channel beyond the last reads the last one's and writes nothing)
  const int length = (count + runs - 1) / runs;
  const int t0 = first + min(run * length, count), t1 = first + min((run + 1) * length, count);
  const int r_column = (mine / part) * 2 * part + mine % part, i_column = r_column + part;
  const int gate_stride = 2 * width;
  const float r_bias = bias[r_column], i_bias = bias[i_column], rate = rates[mine];
  auto step = [&](int t, float& a, float& push) {
    const float r = 1.f / (1.f + expf(-(to_float(gates[(size_t)t * gate_stride + r_column]) + r_bias)));
    const float i = 1.f / (1.f + expf(-(to_float(gates[(size_t)t * gate_stride + i_column]) + i_bias)));
    const float log_a = rate * r;
    a = expf(log_a);
    push = sqrtf(-expm1f(2.f * log_a)) * i * to_float(u[(size_t)t * width + mine]);  // 1 - a^2 without the loss near a = 1
  };
  float* kept = state + (size_t)slots[b] * width + mine;
  float S = *kept;
  if (runs > 1) {
    float A = 1.f, B = 0.f;
    for (int t = t0; t < t1; ++t) {
      float a, push;
      step(t, a, push);
      B = a * B + push;
      A *= a;
    }
    decays[run][threadIdx.x] = A;
    ends[run][threadIdx.x] = B;
    __syncthreads();
    for (int before = 0; before < run; ++before) S = decays[before][threadIdx.x] * S + ends[before][threadIdx.x];
  }
  for (int t = t0; t < t1; ++t) {
    float a, push;
    step(t, a, push);
    S = a * S + push;
    const float z = to_float(branch[(size_t)t * branch_stride + branch_first + mine]);
    const float y = 0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
    if (owns) out[(size_t)t * width + c] = from_float<T>(S * y);
  }
  if (owns && run == runs - 1) *kept = S;
}

// `longest`: the most tokens a request brings.  The branch's activation is gelu_tanh.
extern "C" int llmserve_gated_recurrence(const void* u, int is_float, const void* gates, const float* bias, const float* rates,
                                         const void* branch, int branch_stride, int branch_first, int width, int blocks,
                                         const int* start, const int* slots, int requests, int longest, float* state, void* out,
                                         hipStream_t stream) {
  if (requests <= 0) return 0;
  if (width < 1 || blocks < 1 || width % blocks || branch_first < 0 || branch_first + width > branch_stride) return ERR_BAD_ARGUMENT;
  const int runs = longest <= 8 ? 1 : longest <= 64 ? 4 : MAX_RUNS;
  const dim3 grid(requests, (width + CHANNELS - 1) / CHANNELS), block(CHANNELS, runs);
  if (is_float)
    hipLaunchKernelGGL(gated_recurrence_kernel<float>, grid, block, 0, stream, (const float*)u, (const float*)gates, bias, rates,
                       (const float*)branch, branch_stride, branch_first, width, width / blocks, start, slots, state, (float*)out);
  else
    hipLaunchKernelGGL(gated_recurrence_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)u, (const bf16_t*)gates, bias, rates,
                       (const bf16_t*)branch, branch_stride, branch_first, width, width / blocks, start, slots, state, (bf16_t*)out);
  return LAUNCH_STATUS();
}
