// Several copies of the residual stream side by side (rows of copies * width float32): the copies made from the embedded
// rows, the kernel that does a sublayer's pending write to all copies and reads them for the next sublayer's norm, and a
// weighted sum of two results.
#include "common.h"

#define MAX_COPIES 8

// out[t, s, :] = hidden[t, :] * scale for every copy s
__global__ void stream_copies_kernel(const float* __restrict__ hidden, float* __restrict__ out, int width, int copies, float scale) {
  const size_t t = blockIdx.x;
  for (int h = threadIdx.x; h < width; h += blockDim.x) {
    const float v = hidden[t * width + h] * scale;
    for (int s = 0; s < copies; ++s) out[(t * copies + s) * width + h] = v;
  }
}

extern "C" int llmserve_stream_copies(const float* hidden, float* out, int tokens, int width, int copies, float scale, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (width < 1 || copies < 1) return ERR_BAD_ARGUMENT;
  hipLaunchKernelGGL(stream_copies_kernel, dim3(tokens), dim3(width >= 1024 ? 256 : 64 * ((min(width, 256) + 63) / 64)), 0, stream, hidden, out,
                     width, copies, scale);
  return LAUNCH_STATUS();
}

// One workgroup a row.  With `result` (float32 [parts, tokens, width], its parts added in order): the copies of the row
// become x_t <- sum_s mix[s, t] x_s + write[t] * result, all from the old ones, and go back to memory unless `rows` picks
// the rows (then the copies stay as they are: nobody reads them again).  Then u = sum_s read[s] x_s, and
// out = u * rsqrt(mean(u^2) + eps) * weight.  Everything float32; `out` in the run's type.  A thread takes V neighbouring
// columns at a time (V = 4 where the width allows 16-byte loads), so a row of a few thousand columns is one pass of
// loads that are all in flight together: a step of few rows is as long as its longest workgroup.
template <typename TO, int V>
__global__ __launch_bounds__(1024) void stream_norm_kernel(float* __restrict__ streams, const float* __restrict__ result, int parts,
                                                           size_t part_stride, const float* __restrict__ mix, const float* __restrict__ write,
                                                           const float* __restrict__ read, const void* __restrict__ weight, int weight_is_float,
                                                           TO* __restrict__ out, const int* __restrict__ rows, int width, int copies, float eps) {
  extern __shared__ float summed[];  // [width]: u
  __shared__ float shared[17];
  struct alignas(sizeof(float) * V) Piece { float v[V]; };
  const size_t t = rows ? (size_t)rows[blockIdx.x] : (size_t)blockIdx.x;
  float* mine = streams + t * copies * width;
  float links[MAX_COPIES][MAX_COPIES], outward[MAX_COPIES], inward[MAX_COPIES];
#pragma unroll
  for (int s = 0; s < MAX_COPIES; ++s) {
    inward[s] = s < copies ? read[s] : 0.f;
    outward[s] = (result && s < copies) ? write[s] : 0.f;
#pragma unroll
    for (int d = 0; d < MAX_COPIES; ++d) links[s][d] = (result && s < copies && d < copies) ? mix[s * copies + d] : 0.f;
  }
  float squares = 0.f;
  for (int h = threadIdx.x * V; h < width; h += blockDim.x * V) {
    Piece x[MAX_COPIES];
#pragma unroll
    for (int s = 0; s < MAX_COPIES; ++s) {
      if (s < copies) {
        x[s] = *(const Piece*)(mine + (size_t)s * width + h);
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) x[s].v[j] = 0.f;
      }
    }
    Piece u;
#pragma unroll
    for (int j = 0; j < V; ++j) u.v[j] = 0.f;
    if (result) {
      Piece y;
#pragma unroll
      for (int j = 0; j < V; ++j) y.v[j] = 0.f;
      for (int p = 0; p < parts; ++p) {
        const Piece part = *(const Piece*)(result + p * part_stride + t * width + h);
#pragma unroll
        for (int j = 0; j < V; ++j) y.v[j] += part.v[j];
      }
#pragma unroll
      for (int d = 0; d < MAX_COPIES; ++d) {
        if (d < copies) {
          Piece fresh;
#pragma unroll
          for (int j = 0; j < V; ++j) {
            float sum = 0.f;
#pragma unroll
            for (int s = 0; s < MAX_COPIES; ++s) sum += links[s][d] * x[s].v[j];
            fresh.v[j] = sum + outward[d] * y.v[j];
            u.v[j] += inward[d] * fresh.v[j];
          }
          if (!rows) *(Piece*)(mine + (size_t)d * width + h) = fresh;
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < MAX_COPIES; ++s)
#pragma unroll
        for (int j = 0; j < V; ++j) u.v[j] += inward[s] * x[s].v[j];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      summed[h + j] = u.v[j];
      squares += u.v[j] * u.v[j];
    }
  }
  // every thread goes on with the columns it summed itself; the weights of its first piece are asked for before the
  // workgroup's sum, so that they arrive while it waits
  struct alignas(sizeof(TO) * V) Normed { TO v[V]; };
  const int h0 = threadIdx.x * V;
  float ahead[V];
#pragma unroll
  for (int j = 0; j < V; ++j) ahead[j] = h0 < width ? load_as_float(weight, weight_is_float, h0 + j) : 0.f;
  const float scale = rsqrtf(block_sum(squares, shared) / (float)width + eps);
  for (int h = h0; h < width; h += blockDim.x * V) {
    Normed normed;
#pragma unroll
    for (int j = 0; j < V; ++j)
      normed.v[j] = from_float<TO>(summed[h + j] * scale * (h == h0 ? ahead[j] : load_as_float(weight, weight_is_float, h + j)));
    *(Normed*)(out + (size_t)blockIdx.x * width + h) = normed;
  }
}

extern "C" int llmserve_stream_norm(float* streams, const float* result, int parts, int tokens, const float* mix, const float* write,
                                    const float* read, const void* weight, int weight_is_float, void* out, int out_is_float,
                                    const int* rows, int count, int width, int copies, float eps, hipStream_t stream) {
  if (count <= 0) return 0;
  if (width < 1 || width > 16384 || copies < 1 || copies > MAX_COPIES || (result && (parts < 1 || !mix || !write))) return ERR_BAD_ARGUMENT;
  const size_t lds = (size_t)width * sizeof(float), part_stride = (size_t)tokens * width;
  // 16-byte pieces where every copy of every row starts on a 16-byte border
  const int pieces = width % 4 == 0 ? 4 : 1;
  const int columns = width / pieces;
  const int threads = columns <= 64 ? 64 : min(1024, WAVE * ((columns + WAVE - 1) / WAVE));
#define LAUNCH_STREAM_NORM(TO, V)                                                                                                 \
  hipLaunchKernelGGL((stream_norm_kernel<TO, V>), dim3(count), dim3(threads), lds, stream, streams, result, parts, part_stride, mix, \
                     write, read, weight, weight_is_float, (TO*)out, rows, width, copies, eps)
  if (out_is_float) {
    if (pieces == 4) LAUNCH_STREAM_NORM(float, 4); else LAUNCH_STREAM_NORM(float, 1);
  } else {
    if (pieces == 4) LAUNCH_STREAM_NORM(bf16_t, 4); else LAUNCH_STREAM_NORM(bf16_t, 1);
  }
#undef LAUNCH_STREAM_NORM
  return LAUNCH_STATUS();
}

// out = a_scale * (the parts of a, added in order) + b_scale * (the parts of b); b may be null.  float32 [count].
__global__ void add_scaled_kernel(const float* __restrict__ a, int a_parts, float a_scale, const float* __restrict__ b, int b_parts,
                                  float b_scale, float* __restrict__ out, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float left = 0.f, right = 0.f;
  for (int p = 0; p < a_parts; ++p) left += a[p * count + i];
  if (b)
    for (int p = 0; p < b_parts; ++p) right += b[p * count + i];
  out[i] = a_scale * left + b_scale * right;
}

extern "C" int llmserve_add_scaled(const float* a, int a_parts, float a_scale, const float* b, int b_parts, float b_scale, float* out,
                                   int rows, int width, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (a_parts < 1 || (b && b_parts < 1) || width < 1) return ERR_BAD_ARGUMENT;
  const size_t count = (size_t)rows * width;
  hipLaunchKernelGGL(add_scaled_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, a, a_parts, a_scale, b, b_parts,
                     b_scale, out, count);
  return LAUNCH_STATUS();
}
