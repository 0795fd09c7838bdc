// A gated linear recurrence with a diagonal state.  For channel c of a request's token t:
//   r = sigmoid(gates[t, r_c] + bias[r_c]),  i = sigmoid(gates[t, i_c] + bias[i_c]),  log a = rates[c] * r,
//   S <- a S + sqrt(1 - a^2) * i * u[t, c],   out[t, c] = S * act(branch[t, c])
// where the gates' columns come in `blocks` parts of the channels, a part's r columns before its i columns.  Gates,
// decays and S are float32; u, the gates' products and the branch come in bfloat16 or float32.
//
// The state of a channel meets no other channel.  A workgroup owns CH channels of one request; a long portion is cut
// into as many runs of tokens as the workgroup has rows of threads: every row first walks its run from an empty state and
// notes the product of its decays and what it ends with, then takes the state that the runs before it leave
// (S_end = A S_in + B, run after run) and walks its run again for the results.  The last row leaves the request's state.
// The walk is a chain of dependent steps, each with four exponentials, so its length is what counts: a portion of
// hundreds of tokens goes to workgroups of 16 channels and 64 runs (a run of a 2,048-token prompt is 32 tokens), a step
// of single tokens to workgroups of 64 channels and one run.
#include "common.h"

#define MAX_THREADS 1024

template <typename T, int CH>
__global__ __launch_bounds__(MAX_THREADS) void gated_recurrence_kernel(
    const T* __restrict__ u, const T* __restrict__ gates, const float* __restrict__ bias, const float* __restrict__ rates,
    const T* __restrict__ branch, int branch_stride, int branch_first, int width, int part, const int* __restrict__ start,
    const int* __restrict__ slots, float* __restrict__ state, T* __restrict__ out) {
  __shared__ float decays[MAX_THREADS / CH][CH], ends[MAX_THREADS / CH][CH];
  const int b = blockIdx.x, c = blockIdx.y * CH + threadIdx.x, run = threadIdx.y, runs = blockDim.y;
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
#define LAUNCH_RECURRENCE(T, CH, RUNS)                                                                                            \
  hipLaunchKernelGGL((gated_recurrence_kernel<T, CH>), dim3(requests, (width + CH - 1) / CH), dim3(CH, RUNS), 0, stream, (const T*)u, \
                     (const T*)gates, bias, rates, (const T*)branch, branch_stride, branch_first, width, width / blocks, start,     \
                     slots, state, (T*)out)
#define LAUNCH_RECURRENCE_BY_LENGTH(T)                                                         \
  do {                                                                                         \
    if (longest <= 8) LAUNCH_RECURRENCE(T, 64, 1);                                             \
    else if (longest <= 64) LAUNCH_RECURRENCE(T, 64, 4);                                       \
    else if (longest <= 256) LAUNCH_RECURRENCE(T, 32, 16);                                     \
    else LAUNCH_RECURRENCE(T, 16, 64);                                                         \
  } while (0)
  if (is_float) LAUNCH_RECURRENCE_BY_LENGTH(float); else LAUNCH_RECURRENCE_BY_LENGTH(bf16_t);
#undef LAUNCH_RECURRENCE_BY_LENGTH
#undef LAUNCH_RECURRENCE
  return LAUNCH_STATUS();
}
