// Products whose rows or weights are chosen per tile: a product per head over a run of a row's columns, and the
// products of routed experts over rows that were sorted by expert on the device.  One core: a workgroup of 256
// threads makes a 16 x 64 tile of the result, K in steps of 32 through LDS, float32 arithmetic and sums in the
// order of k whatever the batch holds.  Operands are bfloat16 or float32.  bfloat16 operands whose K is a multiple
// of 32 and whose rows begin at multiples of 8 elements go to the matrix cores instead (the second core below).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define TILE_ROWS 16
#define TILE_COLS 64
#define TILE_K 32
#define PAD_K 33

#define ACT_NONE -1
#define ACT_SILU 0
#define ACT_GELU 1
#define ACT_GELU_TANH 2
#define ACT_RELU 3
// a function of gate and up both, with a limit (gated results only): g = min(gate, limit), u = clamp(up, -limit, limit),
// g * sigmoid(1.702 g) * (u + 1)
#define ACT_LIMITED_SWISH 4

__device__ __forceinline__ float activation_of(int activation, float z) {
  switch (activation) {
    case ACT_NONE: return z;
    case ACT_GELU: return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
    case ACT_GELU_TANH: return 0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
    case ACT_RELU: return fmaxf(z, 0.f);
    default: return z / (1.f + expf(-z));
  }
}

// A code of ACT_GATED or more asks the matrix-core kernels of the experts for a gated result: the product's columns are
// gates and ups in turn (gate_0, up_0, gate_1, ...), and column j of the result, half as wide, is act(gate_j) * up_j,
// both rounded to the result's type first, as they would be if the product were stored and gated by a kernel behind it.
#define ACT_GATED 16

// A lane's four neighbouring columns n0 .. n0 + 3 (n0 a multiple of four) of a row of a product `outputs` wide.
template <typename TO>
__device__ __forceinline__ void store_four(TO* __restrict__ out, size_t row, int n0, int outputs, int activation, const f32x4& v,
                                           float limit = 0.f) {
  if (activation < ACT_GATED) {
    TO* dst = out + row * outputs;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n0 + i < outputs) dst[n0 + i] = from_float<TO>(activation_of(activation, v[i]));
    return;
  }
  TO* dst = out + row * (outputs / 2);
#pragma unroll
  for (int pair = 0; pair < 2; ++pair) {
    const int n = n0 + 2 * pair;
    if (n + 1 < outputs) {
      const float gate = to_float(from_float<TO>(v[2 * pair])), up = to_float(from_float<TO>(v[2 * pair + 1]));
      if (activation - ACT_GATED == ACT_LIMITED_SWISH) {
        const float g = fminf(gate, limit), u = fminf(fmaxf(up, -limit), limit);
        dst[n / 2] = from_float<TO>(g / (1.f + expf(-1.702f * g)) * (u + 1.f));
      } else {
        dst[n / 2] = from_float<TO>(activation_of(activation - ACT_GATED, gate) * up);
      }
    }
  }
}

// Thread t loads two elements of x row t / 16 and eight of weight row t / 4 per step, and owns the results
// (row t / 16, columns t % 16 + 16 j).  `x_row` / `w_row` are the thread's rows to load (null: zeros).
template <typename TX, typename TW>
__device__ __forceinline__ void tile_product(const TX* x_row, const TW* w_row, int inner, float (&acc)[4], float* xs, float* ws) {
  const int t = threadIdx.x, r = t / 16, g = t % 16;
  const int xk = (t % 16) * 2, wn = t / 4, wk = (t % 4) * 8;
  for (int k0 = 0; k0 < inner; k0 += TILE_K) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int k = k0 + xk + e;
      xs[r * PAD_K + xk + e] = (x_row && k < inner) ? to_float(x_row[k]) : 0.f;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = k0 + wk + e;
      ws[wn * PAD_K + wk + e] = (w_row && k < inner) ? to_float(w_row[k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TILE_K; ++kk) {
      const float a = xs[r * PAD_K + kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] += a * ws[(g + 16 * j) * PAD_K + kk];
    }
    __syncthreads();
  }
}

// The matrix-core form.  A wave makes NT x MT tiles of v_mfma_f32_16x16x32_bf16: weight rows are the A operand (lane l
// holds row l % 16, k = (l / 16) * 8 .. + 8 of a 32-wide step), the operand's rows the B operand (lane l: row l % 16, the
// same k), both straight from memory in 16-byte loads, and the result tile D[n][m] leaves four consecutive n of row
// l % 16 in lane l.  `w_row[s]` and `x_row[t]` are the lane's rows already moved to its k (null: zeros).
template <int NT, int MT>
__device__ __forceinline__ void tile_product_mfma(const bf16_t* const (&w_row)[NT], const bf16_t* const (&x_row)[MT], int inner,
                                                  f32x4 (&acc)[NT][MT]) {
  const bf16x8 zero = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll(NT * MT <= 2 ? 8 : 4)
  for (int k0 = 0; k0 < inner; k0 += 32) {
    bf16x8 a[NT], b[MT];
#pragma unroll
    for (int s = 0; s < NT; ++s) a[s] = w_row[s] ? *(const bf16x8*)(w_row[s] + k0) : zero;
#pragma unroll
    for (int t = 0; t < MT; ++t) b[t] = x_row[t] ? *(const bf16x8*)(x_row[t] + k0) : zero;
#pragma unroll
    for (int s = 0; s < NT; ++s)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s], b[t], acc[s][t], 0, 0, 0);
  }
}

// A workgroup of four waves makes 16 MT rows by 64 NT columns, wave v the columns 16 NT v .. + 16 NT.
template <int NT, int MT>
__global__ __launch_bounds__(256) void headwise_mfma_kernel(const bf16_t* __restrict__ x, int x_stride, int first, int head_stride,
                                                            const bf16_t* __restrict__ w, int outputs, int inner,
                                                            bf16_t* __restrict__ out, int out_stride, int out_first,
                                                            int out_head_stride, int rows) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int head = blockIdx.z, row0 = blockIdx.y * 16 * MT, col0 = (blockIdx.x * 4 + wave) * 16 * NT;
  if (col0 >= outputs) return;
  const bf16_t* w_row[NT];
  const bf16_t* x_row[MT];
#pragma unroll
  for (int s = 0; s < NT; ++s) {
    const int n = col0 + s * 16 + r;
    w_row[s] = n < outputs ? w + ((size_t)head * outputs + n) * inner + g * 8 : nullptr;
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = row0 + t * 16 + r;
    x_row[t] = m < rows ? x + (size_t)m * x_stride + first + (size_t)head * head_stride + g * 8 : nullptr;
  }
  f32x4 acc[NT][MT];
#pragma unroll
  for (int s = 0; s < NT; ++s)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[s][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  tile_product_mfma<NT, MT>(w_row, x_row, inner, acc);
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = row0 + t * 16 + r;
    if (m >= rows) continue;
    bf16_t* dst = out + (size_t)m * out_stride + out_first + (size_t)head * out_head_stride;
#pragma unroll
    for (int s = 0; s < NT; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = col0 + s * 16 + g * 4 + i;
        if (n < outputs) dst[n] = (bf16_t)acc[s][t][i];
      }
  }
}

template <int NT, int MT, typename TO>
__global__ __launch_bounds__(256) void expert_product_mfma_kernel(const bf16_t* __restrict__ x, const int* __restrict__ order, int top,
                                                                  const bf16_t* __restrict__ w, int outputs, int inner,
                                                                  const int* __restrict__ tiles, TO* __restrict__ out, int activation, float limit) {
  const int* tile = tiles + 3 * (size_t)blockIdx.y;
  const int expert = tile[0], first = tile[1], rows = tile[2];
  if (rows == 0) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int col0 = (blockIdx.x * 4 + wave) * 16 * NT;
  if (col0 >= outputs) return;
  const bf16_t* w_row[NT];
  const bf16_t* x_row[MT];
#pragma unroll
  for (int s = 0; s < NT; ++s) {
    const int n = col0 + s * 16 + r;
    w_row[s] = n < outputs ? w + ((size_t)expert * outputs + n) * inner + g * 8 : nullptr;
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    x_row[t] = nullptr;
    if (m < rows) {
      const int place = first + m;
      x_row[t] = x + (size_t)(top > 0 ? order[place] / top : place) * inner + g * 8;
    }
  }
  f32x4 acc[NT][MT];
#pragma unroll
  for (int s = 0; s < NT; ++s)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[s][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  tile_product_mfma<NT, MT>(w_row, x_row, inner, acc);
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + r;
    if (m >= rows) continue;
#pragma unroll
    for (int s = 0; s < NT; ++s) store_four<TO>(out, (size_t)(first + m), col0 + s * 16 + g * 4, outputs, activation, acc[s][t], limit);
  }
}

// The experts' products of a step of many rows (prompts): tiles of 128 rows of one expert by 128 columns, K in steps of 64
// through LDS.  All 256 threads bring the two operand tiles from memory sixteen bytes at a time, eight threads a row (128
// bytes in a row, where the kernel above asks for sixteen rows of 64 bytes an instruction and is bound by the address
// path), two steps ahead in registers; the four waves (2 x 2) each make 64 x 64 of the result out of LDS.  Rows of LDS are
// 144 bytes apart (banks).  Rows and columns beyond the tile's are read from the last valid one and never stored.
#define TILED_ROWS 128
#define TILED_K 64
#define TILED_LINE 72  // elements: 64 and 8 of padding
template <typename TO>
__global__ __launch_bounds__(256) void expert_tiled_kernel(const bf16_t* __restrict__ x, const int* __restrict__ order, int top,
                                                           const bf16_t* __restrict__ w, int outputs, int inner,
                                                           const int* __restrict__ tiles, TO* __restrict__ out, int activation, float limit) {
  __shared__ __attribute__((aligned(16))) bf16_t xs[TILED_ROWS * TILED_LINE], ws[TILED_ROWS * TILED_LINE];
  const int* tile = tiles + 3 * (size_t)blockIdx.y;
  const int expert = tile[0], first = tile[1], rows = tile[2];
  if (rows == 0) return;
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63, r = lane & 15, g = lane >> 4;
  const int wave_row = (wave >> 1) * 64, wave_col = (wave & 1) * 64;
  const int col0 = blockIdx.x * TILED_ROWS;
  const int piece = t % 8;  // which sixteen bytes of a row's 128 a step
  const bf16_t* x_from[4];
  const bf16_t* w_from[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = min(t / 8 + 32 * j, rows - 1), place = first + row;
    x_from[j] = x + (size_t)(top > 0 ? order[place] / top : place) * inner + piece * 8;
    const int n = min(col0 + t / 8 + 32 * j, outputs - 1);
    w_from[j] = w + ((size_t)expert * outputs + n) * inner + piece * 8;
  }
  bf16x8 x_next[4], w_next[4], x_after[4], w_after[4];  // the next step's pieces, and the one's after it
  const int second = min(TILED_K, inner - TILED_K);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    x_next[j] = *(const bf16x8*)x_from[j];
    w_next[j] = *(const bf16x8*)w_from[j];
    x_after[j] = *(const bf16x8*)(x_from[j] + second);
    w_after[j] = *(const bf16x8*)(w_from[j] + second);
  }
  f32x4 acc[4][4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int u = 0; u < 4; ++u) acc[s][u] = (f32x4){0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < inner; k0 += TILED_K) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      *(bf16x8*)&xs[(t / 8 + 32 * j) * TILED_LINE + piece * 8] = x_next[j];
      *(bf16x8*)&ws[(t / 8 + 32 * j) * TILED_LINE + piece * 8] = w_next[j];
      x_next[j] = x_after[j];
      w_next[j] = w_after[j];
    }
    __syncthreads();
    const int ahead = min(k0 + 2 * TILED_K, inner - TILED_K);  // (in no branch; the last steps ask for the last again)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      x_after[j] = *(const bf16x8*)(x_from[j] + ahead);
      w_after[j] = *(const bf16x8*)(w_from[j] + ahead);
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      bf16x8 a[4], b[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) a[s] = *(const bf16x8*)&ws[(wave_col + s * 16 + r) * TILED_LINE + half * 32 + g * 8];
#pragma unroll
      for (int u = 0; u < 4; ++u) b[u] = *(const bf16x8*)&xs[(wave_row + u * 16 + r) * TILED_LINE + half * 32 + g * 8];
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int u = 0; u < 4; ++u) acc[s][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s], b[u], acc[s][u], 0, 0, 0);
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int m = wave_row + u * 16 + r;
    if (m >= rows) continue;
#pragma unroll
    for (int s = 0; s < 4; ++s) store_four<TO>(out, (size_t)(first + m), col0 + wave_col + s * 16 + g * 4, outputs, activation, acc[s][u], limit);
  }
}

// The experts' products of a step of few rows (decoding): every tile holds a few rows of one expert, and the product is a
// stream of that expert's weights.  A workgroup owns 16 weight rows of one tile's expert and its four waves take the
// 32-wide steps of K in turn (wave v the steps v, v + 4, ...), so that four times as many loads are under way as with a
// wave a tile of weight rows; the waves' partial tiles are added through LDS in wave order.
template <typename TO>
__global__ __launch_bounds__(256) void expert_stream_kernel(const bf16_t* __restrict__ x, const int* __restrict__ order, int top,
                                                            const bf16_t* __restrict__ w, int outputs, int inner,
                                                            const int* __restrict__ tiles, TO* __restrict__ out, int activation, float limit) {
  __shared__ f32x4 partial[4][WAVE];
  const int* tile = tiles + 3 * (size_t)blockIdx.y;
  const int expert = tile[0], first = tile[1], rows = tile[2];
  if (rows == 0) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int n = min((int)blockIdx.x * 16 + r, outputs - 1);
  const bf16_t* w_row = w + ((size_t)expert * outputs + n) * inner + g * 8;
  const bf16_t* x_row = nullptr;
  if (r < rows) {
    const int place = first + r;
    x_row = x + (size_t)(top > 0 ? order[place] / top : place) * inner + g * 8;
  }
  const bf16x8 zero = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
  f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
  const int steps = inner / 32;
#pragma unroll 4
  for (int step = wave; step < steps; step += 4) {
    const bf16x8 a = *(const bf16x8*)(w_row + step * 32);
    const bf16x8 b = x_row ? *(const bf16x8*)(x_row + step * 32) : zero;
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
  }
  partial[wave][lane] = acc;
  __syncthreads();
  if (wave != 0 || r >= rows) return;
  f32x4 total = partial[0][lane];
#pragma unroll
  for (int v = 1; v < 4; ++v) total += partial[v][lane];
  store_four<TO>(out, (size_t)(first + r), blockIdx.x * 16 + g * 4, outputs, activation, total, limit);
}

// ---------------------------------------------------------------------------- a product per head
// out[t, out_first + h * out_head_stride + n] = sum_k x[t, first + h * head_stride + k] * w[h, n, k]
template <typename T>
__global__ __launch_bounds__(256) void headwise_kernel(const T* __restrict__ x, int x_stride, int first, int head_stride,
                                                       const T* __restrict__ w, int outputs, int inner, T* __restrict__ out,
                                                       int out_stride, int out_first, int out_head_stride, int rows) {
  __shared__ float xs[TILE_ROWS * PAD_K], ws[TILE_COLS * PAD_K];
  const int head = blockIdx.z, row0 = blockIdx.y * TILE_ROWS, col0 = blockIdx.x * TILE_COLS;
  const int t = threadIdx.x;
  const int load_row = row0 + t / 16, load_col = col0 + t / 4;
  const T* x_row = load_row < rows ? x + (size_t)load_row * x_stride + first + (size_t)head * head_stride : nullptr;
  const T* w_row = load_col < outputs ? w + ((size_t)head * outputs + load_col) * inner : nullptr;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  tile_product(x_row, w_row, inner, acc, xs, ws);
  const int row = row0 + t / 16;
  if (row >= rows) return;
  T* dst = out + (size_t)row * out_stride + out_first + (size_t)head * out_head_stride;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = col0 + t % 16 + 16 * j;
    if (n < outputs) dst[n] = from_float<T>(acc[j]);
  }
}

extern "C" int llmserve_headwise_linear(const void* x, int is_float, int rows, int x_stride, int first, int head_stride,
                                        const void* w, int heads, int outputs, int inner, void* out, int out_stride,
                                        int out_first, int out_head_stride, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (heads < 1 || outputs < 1 || inner < 1 || first + (heads - 1) * head_stride + inner > x_stride ||
      out_first + (heads - 1) * out_head_stride + outputs > out_stride || heads > 65535)
    return ERR_BAD_ARGUMENT;
  const dim3 grid((outputs + TILE_COLS - 1) / TILE_COLS, (rows + TILE_ROWS - 1) / TILE_ROWS, heads);
  if (grid.y > 65535) return ERR_BAD_ARGUMENT;
  if (!is_float && inner % 32 == 0 && x_stride % 8 == 0 && first % 8 == 0 && head_stride % 8 == 0) {
    // the matrix cores: four row tiles a wave for many rows, one for a few; as many column tiles as the columns need
    const int mt = rows > 16 ? 4 : 1, nt = outputs <= 64 ? 1 : outputs <= 128 ? 2 : 4;
    const dim3 cores((outputs + 64 * nt - 1) / (64 * nt), (rows + 16 * mt - 1) / (16 * mt), heads);
#define LAUNCH_HEADWISE(NT, MT)                                                                                                 \
  hipLaunchKernelGGL((headwise_mfma_kernel<NT, MT>), cores, dim3(256), 0, stream, (const bf16_t*)x, x_stride, first, head_stride, \
                     (const bf16_t*)w, outputs, inner, (bf16_t*)out, out_stride, out_first, out_head_stride, rows)
    if (mt == 4) {
      if (nt == 1) LAUNCH_HEADWISE(1, 4); else if (nt == 2) LAUNCH_HEADWISE(2, 4); else LAUNCH_HEADWISE(4, 4);
    } else {
      if (nt == 1) LAUNCH_HEADWISE(1, 1); else if (nt == 2) LAUNCH_HEADWISE(2, 1); else LAUNCH_HEADWISE(4, 1);
    }
#undef LAUNCH_HEADWISE
    return LAUNCH_STATUS();
  }
  if (is_float)
    hipLaunchKernelGGL(headwise_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, x_stride, first, head_stride,
                       (const float*)w, outputs, inner, (float*)out, out_stride, out_first, out_head_stride, rows);
  else
    hipLaunchKernelGGL(headwise_kernel<bf16_t>, grid, dim3(256), 0, stream, (const bf16_t*)x, x_stride, first, head_stride,
                       (const bf16_t*)w, outputs, inner, (bf16_t*)out, out_stride, out_first, out_head_stride, rows);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- routing
// One wave a token: s_e = sigmoid(z[t, e]) or softmax(z[t, :])_e; the `top` experts with the largest s_e + correction_e,
// the lower index first among equals, taken from the experts of the `keep` best of `groups` equal groups of neighbours;
// chosen[t, i] and weight[t, i] = scale * s_e, with `renormalise` scale * s_e / (sum of the chosen s + 1e-20).  Lane l
// keeps the experts l, l + 64, ...; a pick is the wave's best of the lanes' best, which is then struck out.
#define ROUTE_PER_LANE 16
__global__ __launch_bounds__(WAVE) void route_kernel(const float* __restrict__ z, int z_stride, int experts,
                                                     const float* __restrict__ correction, int top, float scale,
                                                     int* __restrict__ chosen, float* __restrict__ weight, int softmax,
                                                     int groups, int keep, int renormalise) {
  __shared__ float by_expert[ROUTE_PER_LANE * WAVE];
  __shared__ float by_group[ROUTE_PER_LANE * WAVE];
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* row = z + (size_t)t * z_stride;
  float score[ROUTE_PER_LANE], choice[ROUTE_PER_LANE];
  float top_z = -INFINITY, total = 1.f;
  if (softmax) {  // over all experts: exp(z - max) / sum
#pragma unroll
    for (int j = 0; j < ROUTE_PER_LANE; ++j) {
      const int e = lane + j * WAVE;
      if (e < experts) top_z = fmaxf(top_z, row[e]);
    }
    top_z = wave_max(top_z);
    total = 0.f;
#pragma unroll
    for (int j = 0; j < ROUTE_PER_LANE; ++j) {
      const int e = lane + j * WAVE;
      score[j] = e < experts ? expf(row[e] - top_z) : 0.f;
      total += score[j];
    }
    total = wave_sum(total);
  }
#pragma unroll
  for (int j = 0; j < ROUTE_PER_LANE; ++j) {
    const int e = lane + j * WAVE;
    if (softmax) score[j] = score[j] / total;
    else score[j] = e < experts ? 1.f / (1.f + expf(-row[e])) : 0.f;
    choice[j] = e < experts ? score[j] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  if (groups > 1) {
    // Only the experts of the `keep` best groups of neighbours stay; a group's score is its largest (the lower index
    // among equals, as everywhere here).
    const int size = experts / groups;
#pragma unroll
    for (int j = 0; j < ROUTE_PER_LANE; ++j)
      if (lane + j * WAVE < experts) by_expert[lane + j * WAVE] = choice[j];
    __syncthreads();
    for (int g = lane; g < groups; g += WAVE) {
      float best = -INFINITY;
      for (int i = 0; i < size; ++i) best = fmaxf(best, by_expert[g * size + i]);
      by_group[g] = best;
    }
    __syncthreads();
    // group g stays if fewer than `keep` groups come before it in the order (score descending, index ascending)
#pragma unroll
    for (int j = 0; j < ROUTE_PER_LANE; ++j) {
      const int e = lane + j * WAVE;
      if (e >= experts) continue;
      const int g = e / size;
      const float mine = by_group[g];
      int before = 0;
      for (int o = 0; o < groups; ++o) before += (by_group[o] > mine || (by_group[o] == mine && o < g)) ? 1 : 0;
      if (before >= keep) choice[j] = -INFINITY;
    }
  }
  float sum = 0.f;
  for (int i = 0; i < top; ++i) {
    float best = -INFINITY, best_score = 0.f;
    int best_expert = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < ROUTE_PER_LANE; ++j) {
      const int e = lane + j * WAVE;
      if (e < experts && (choice[j] > best || best_expert == 0x7fffffff)) { best = choice[j]; best_score = score[j]; best_expert = e; }
    }
#pragma unroll
    for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
      const float other = __shfl_xor(best, offset, WAVE), other_score = __shfl_xor(best_score, offset, WAVE);
      const int other_expert = __shfl_xor(best_expert, offset, WAVE);
      if (other_expert != 0x7fffffff && (best_expert == 0x7fffffff || other > best || (other == best && other_expert < best_expert))) {
        best = other; best_score = other_score; best_expert = other_expert;
      }
    }
    sum += best_score;
    if (lane == 0) {
      chosen[(size_t)t * top + i] = best_expert;
      weight[(size_t)t * top + i] = renormalise ? best_score : scale * best_score;
    }
#pragma unroll
    for (int j = 0; j < ROUTE_PER_LANE; ++j)
      if (lane + j * WAVE == best_expert) choice[j] = -INFINITY;
  }
  if (renormalise && lane == 0)  // (the lane reads back what it wrote itself)
    for (int i = 0; i < top; ++i) weight[(size_t)t * top + i] = weight[(size_t)t * top + i] / (sum + 1e-20f) * scale;
}

// `correction` may be null (the choice is by score alone).  softmax 0: sigmoid of each score; 1: softmax over all experts.
extern "C" int llmserve_route(const float* z, int z_stride, int experts, const float* correction, int top, float scale,
                              int* chosen, float* weight, int tokens, int softmax, int groups, int keep, int renormalise,
                              hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (experts < 1 || top < 1 || top > experts || experts > z_stride || experts > ROUTE_PER_LANE * WAVE) return ERR_BAD_ARGUMENT;
  if (groups < 1 || experts % groups || keep < 1 || keep > groups || top > keep * (experts / groups)) return ERR_BAD_ARGUMENT;
  hipLaunchKernelGGL(route_kernel, dim3(tokens), dim3(WAVE), 0, stream, z, z_stride, experts, correction, top, scale, chosen, weight,
                     softmax, groups, keep, renormalise);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- sorting the (token, choice) pairs by expert
// One workgroup.  place[p] is where pair p = t * top + i stands in the order by expert (the order within an expert is
// whichever the counting gave: every row is computed by itself, so results do not depend on it); order[place[p]] = p.
// The tiles of the grouped products, up to `tile_rows` rows of one expert each: tile[i] = (expert, first place, rows);
// there is room for ceil(pairs / tile_rows) + experts of them, and those not needed have no rows.
#define SORT_THREADS 1024
#define MAX_EXPERTS 1024
__global__ __launch_bounds__(SORT_THREADS) void sort_pairs_kernel(const int* __restrict__ chosen, int pairs, int experts,
                                                                  int* __restrict__ place, int* __restrict__ order,
                                                                  int* __restrict__ tiles, int capacity, int tile_rows) {
  __shared__ int count[MAX_EXPERTS], first[MAX_EXPERTS], first_tile[MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < experts; e += SORT_THREADS) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += SORT_THREADS) place[p] = atomicAdd(&count[chosen[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int rows = 0, tile = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = rows;
      first_tile[e] = tile;
      rows += count[e];
      tile += (count[e] + tile_rows - 1) / tile_rows;
    }
    first_tile[experts] = tile;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < pairs; p += SORT_THREADS) {
    const int where = first[chosen[p]] + place[p];
    place[p] = where;
    order[where] = p;
  }
  for (int e = threadIdx.x; e < experts; e += SORT_THREADS) {
    const int n = (count[e] + tile_rows - 1) / tile_rows;
    for (int i = 0; i < n; ++i) {
      int* tile = tiles + 3 * (size_t)(first_tile[e] + i);
      tile[0] = e;
      tile[1] = first[e] + i * tile_rows;
      tile[2] = min(tile_rows, count[e] - i * tile_rows);
    }
  }
  for (int i = first_tile[experts] + threadIdx.x; i < capacity; i += SORT_THREADS) {
    tiles[3 * (size_t)i] = 0;
    tiles[3 * (size_t)i + 1] = 0;
    tiles[3 * (size_t)i + 2] = 0;
  }
}

extern "C" int llmserve_sort_pairs(const int* chosen, int pairs, int experts, int* place, int* order, int* tiles,
                                   int capacity, int tile_rows, hipStream_t stream) {
  if (pairs <= 0) return 0;
  if (experts < 1 || experts > MAX_EXPERTS || (tile_rows != 16 && tile_rows != 64 && tile_rows != 128) ||
      capacity < (pairs + tile_rows - 1) / tile_rows + experts)
    return ERR_BAD_ARGUMENT;
  hipLaunchKernelGGL(sort_pairs_kernel, dim3(1), dim3(SORT_THREADS), 0, stream, chosen, pairs, experts, place, order, tiles, capacity,
                     tile_rows);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- the experts' products
// Tile i of the list holds `rows` rows of expert e from place `first` on.  With `top` > 0 the operand's rows are the
// tokens' (row order[place] / top of x: the first product of an expert); with top = 0 they are the places' own (the
// second).  out[place, n] = act(sum_k row[k] * w[e, n, k]).
template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void expert_product_kernel(const TX* __restrict__ x, const int* __restrict__ order, int top,
                                                             const TW* __restrict__ w, int outputs, int inner,
                                                             const int* __restrict__ tiles, TO* __restrict__ out, int activation) {
  __shared__ float xs[TILE_ROWS * PAD_K], ws[TILE_COLS * PAD_K];
  const int* tile = tiles + 3 * (size_t)blockIdx.y;
  const int expert = tile[0], first = tile[1], rows = tile[2];
  if (rows == 0) return;  // (the whole workgroup: nothing waits)
  const int t = threadIdx.x, col0 = blockIdx.x * TILE_COLS;
  const int load_row = t / 16, load_col = col0 + t / 4;
  const TX* x_row = nullptr;
  if (load_row < rows) {
    const int place = first + load_row;
    x_row = x + (size_t)(top > 0 ? order[place] / top : place) * inner;
  }
  const TW* w_row = load_col < outputs ? w + ((size_t)expert * outputs + load_col) * inner : nullptr;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  tile_product(x_row, w_row, inner, acc, xs, ws);
  if (t / 16 >= rows) return;
  TO* dst = out + (size_t)(first + t / 16) * outputs;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = col0 + t % 16 + 16 * j;
    if (n < outputs) dst[n] = from_float<TO>(activation_of(activation, acc[j]));
  }
}

// x, w and the first product's result are of one type (bfloat16 or float32); the second product's result is float32.
// `tile_rows` is what the tiles were made for: 16; or, bfloat16 on the matrix cores only, 64 (K in steps of 32) or 128 (K in
// steps of 64: operands through LDS).
// Whether the product of these operands runs on a kernel that can gate its result (ACT_GATED).
extern "C" int llmserve_expert_product_gates(int is_float, int inner, int tile_rows) {
  if (is_float) return 0;
  return tile_rows == TILED_ROWS ? inner % TILED_K == 0 : inner % 32 == 0;
}

extern "C" int llmserve_expert_product(const void* x, int is_float, const int* order, int top, const void* w, int outputs,
                                       int inner, const int* tiles, int capacity, int tile_rows, void* out, int out_is_float,
                                       int activation, float limit, hipStream_t stream) {
  if (capacity <= 0) return 0;
  if ((activation == ACT_GATED + ACT_LIMITED_SWISH && !(limit > 0.f)) || activation == ACT_LIMITED_SWISH) return ERR_BAD_ARGUMENT;
  if (capacity > 65535 || outputs < 1 || inner < 1) return ERR_BAD_ARGUMENT;
  // a gated result comes from the matrix-core kernels alone, of an even number of columns
  if (activation >= ACT_GATED && (outputs % 2 || !llmserve_expert_product_gates(is_float, inner, tile_rows))) return ERR_BAD_ARGUMENT;
  if (!is_float && tile_rows == TILED_ROWS) {
    if (inner % TILED_K) return ERR_BAD_ARGUMENT;
    const dim3 through_lds((outputs + TILED_ROWS - 1) / TILED_ROWS, capacity);
    if (out_is_float)
      hipLaunchKernelGGL(expert_tiled_kernel<float>, through_lds, dim3(256), 0, stream, (const bf16_t*)x, order, top, (const bf16_t*)w,
                         outputs, inner, tiles, (float*)out, activation, limit);
    else
      hipLaunchKernelGGL(expert_tiled_kernel<bf16_t>, through_lds, dim3(256), 0, stream, (const bf16_t*)x, order, top, (const bf16_t*)w,
                         outputs, inner, tiles, (bf16_t*)out, activation, limit);
    return LAUNCH_STATUS();
  }
  if (!is_float && inner % 32 == 0) {
    if (tile_rows == 16 && capacity * ((outputs + 15) / 16) <= 8192) {
      // a few tiles (decoding) stream their experts' weights: sixteen weight rows a workgroup, K dealt out to its waves
      const dim3 streams((outputs + 15) / 16, capacity);
      if (out_is_float)
        hipLaunchKernelGGL(expert_stream_kernel<float>, streams, dim3(256), 0, stream, (const bf16_t*)x, order, top, (const bf16_t*)w,
                           outputs, inner, tiles, (float*)out, activation, limit);
      else
        hipLaunchKernelGGL(expert_stream_kernel<bf16_t>, streams, dim3(256), 0, stream, (const bf16_t*)x, order, top, (const bf16_t*)w,
                           outputs, inner, tiles, (bf16_t*)out, activation, limit);
      return LAUNCH_STATUS();
    }
    const int nt = outputs <= 64 ? 1 : outputs <= 128 ? 2 : 4;
    const dim3 cores((outputs + 64 * nt - 1) / (64 * nt), capacity);
#define LAUNCH_EXPERTS(NT, MT)                                                                                                  \
  do {                                                                                                                          \
    if (out_is_float)                                                                                                           \
      hipLaunchKernelGGL((expert_product_mfma_kernel<NT, MT, float>), cores, dim3(256), 0, stream, (const bf16_t*)x, order, top, \
                         (const bf16_t*)w, outputs, inner, tiles, (float*)out, activation, limit);                              \
    else                                                                                                                        \
      hipLaunchKernelGGL((expert_product_mfma_kernel<NT, MT, bf16_t>), cores, dim3(256), 0, stream, (const bf16_t*)x, order, top, \
                         (const bf16_t*)w, outputs, inner, tiles, (bf16_t*)out, activation, limit);                             \
  } while (0)
    if (tile_rows == 64) {
      if (nt == 1) LAUNCH_EXPERTS(1, 4); else if (nt == 2) LAUNCH_EXPERTS(2, 4); else LAUNCH_EXPERTS(4, 4);
    } else if (tile_rows == 16) {
      if (nt == 1) LAUNCH_EXPERTS(1, 1); else if (nt == 2) LAUNCH_EXPERTS(2, 1); else LAUNCH_EXPERTS(4, 1);
    } else {
      return ERR_BAD_ARGUMENT;
    }
#undef LAUNCH_EXPERTS
    return LAUNCH_STATUS();
  }
  if (tile_rows != TILE_ROWS) return ERR_BAD_ARGUMENT;
  const dim3 grid((outputs + TILE_COLS - 1) / TILE_COLS, capacity);
  if (is_float) {
    if (!out_is_float) return ERR_BAD_ARGUMENT;
    hipLaunchKernelGGL((expert_product_kernel<float, float, float>), grid, dim3(256), 0, stream, (const float*)x, order, top,
                       (const float*)w, outputs, inner, tiles, (float*)out, activation);
  } else if (out_is_float) {
    hipLaunchKernelGGL((expert_product_kernel<bf16_t, bf16_t, float>), grid, dim3(256), 0, stream, (const bf16_t*)x, order, top,
                       (const bf16_t*)w, outputs, inner, tiles, (float*)out, activation);
  } else {
    hipLaunchKernelGGL((expert_product_kernel<bf16_t, bf16_t, bf16_t>), grid, dim3(256), 0, stream, (const bf16_t*)x, order, top,
                       (const bf16_t*)w, outputs, inner, tiles, (bf16_t*)out, activation);
  }
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- the tokens' weighted sums
// out[t] = sum_i weight[t, i] * rows[place[t * top + i]], in the order of i; with `shared`, plus
// sigmoid(gates[t, gate_column]) * shared[t] (an expert that every token uses, behind a gate of its own).
__global__ void combine_pairs_kernel(const float* __restrict__ rows, const int* __restrict__ place, const float* __restrict__ weight,
                                     int top, float* __restrict__ out, int width, const float* __restrict__ shared,
                                     const float* __restrict__ gates, int gate_stride, int gate_column) {
  const int t = blockIdx.x;
  const float gate = shared ? (gates ? 1.f / (1.f + expf(-gates[(size_t)t * gate_stride + gate_column])) : 1.f) : 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float sum = 0.f;
    for (int i = 0; i < top; ++i) sum += weight[(size_t)t * top + i] * rows[(size_t)place[(size_t)t * top + i] * width + c];
    if (shared) sum += gate * shared[(size_t)t * width + c];
    out[(size_t)t * width + c] = sum;
  }
}

extern "C" int llmserve_combine_pairs(const float* rows, const int* place, const float* weight, int top, float* out, int tokens,
                                      int width, const float* shared, const float* gates, int gate_stride, int gate_column,
                                      hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (shared && gates && (gate_column < 0 || gate_column >= gate_stride)) return ERR_BAD_ARGUMENT;  // (no gates: the shared rows are added as they are)
  hipLaunchKernelGGL(combine_pairs_kernel, dim3(tokens), dim3(256), 0, stream, rows, place, weight, top, out, width, shared, gates,
                     gate_stride, gate_column);
  return LAUNCH_STATUS();
}
