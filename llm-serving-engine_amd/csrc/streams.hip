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
// out = u * rsqrt(mean(u^2) + eps) * weight.  Everything float32; `out` in the run's type.
template <typename TO>
__global__ __launch_bounds__(256) void stream_norm_kernel(float* __restrict__ streams, const float* __restrict__ result, int parts,
                                                          size_t part_stride, const float* __restrict__ mix, const float* __restrict__ write,
                                                          const float* __restrict__ read, const void* __restrict__ weight, int weight_is_float,
                                                          TO* __restrict__ out, const int* __restrict__ rows, int width, int copies, float eps) {
  extern __shared__ float summed[];  // [width]: u
  __shared__ float shared[17];
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
  for (int h = threadIdx.x; h < width; h += blockDim.x) {
    float x[MAX_COPIES];
#pragma unroll
    for (int s = 0; s < MAX_COPIES; ++s) x[s] = s < copies ? mine[(size_t)s * width + h] : 0.f;
    float u = 0.f;
    if (result) {
      float y = 0.f;
      for (int p = 0; p < parts; ++p) y += result[p * part_stride + t * width + h];
#pragma unroll
      for (int d = 0; d < MAX_COPIES; ++d) {
        if (d < copies) {
          float fresh = 0.f;
#pragma unroll
          for (int s = 0; s < MAX_COPIES; ++s) fresh += links[s][d] * x[s];
          fresh += outward[d] * y;
          if (!rows) mine[(size_t)d * width + h] = fresh;
          u += inward[d] * fresh;
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < MAX_COPIES; ++s) u += inward[s] * x[s];
    }
    summed[h] = u;
    squares += u * u;
  }
  const float scale = rsqrtf(block_sum(squares, shared) / (float)width + eps);
  for (int h = threadIdx.x; h < width; h += blockDim.x)
    out[(size_t)blockIdx.x * width + h] = from_float<TO>(summed[h] * scale * load_as_float(weight, weight_is_float, h));
}

extern "C" int llmserve_stream_norm(float* streams, const float* result, int parts, int tokens, const float* mix, const float* write,
                                    const float* read, const void* weight, int weight_is_float, void* out, int out_is_float,
                                    const int* rows, int count, int width, int copies, float eps, hipStream_t stream) {
  if (count <= 0) return 0;
  if (width < 1 || width > 16384 || copies < 1 || copies > MAX_COPIES || (result && (parts < 1 || !mix || !write))) return ERR_BAD_ARGUMENT;
  const size_t lds = (size_t)width * sizeof(float), part_stride = (size_t)tokens * width;
  const int threads = width <= 64 ? 64 : width <= 128 ? 128 : 256;
  if (out_is_float)
    hipLaunchKernelGGL(stream_norm_kernel<float>, dim3(count), dim3(threads), lds, stream, streams, result, parts, part_stride, mix, write,
                       read, weight, weight_is_float, (float*)out, rows, width, copies, eps);
  else
    hipLaunchKernelGGL(stream_norm_kernel<bf16_t>, dim3(count), dim3(threads), lds, stream, streams, result, parts, part_stride, mix, write,
                       read, weight, weight_is_float, (bf16_t*)out, rows, width, copies, eps);
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
