// Operations around attention heads and around norms that act on a sublayer's result:
//   stream_rows     hidden += delta; the rows in the run dtype
//   add_normed      hidden += rms_norm(update) * weight; the rows in the run dtype, or, with the weight of a next norm,
//                   rms_norm(hidden) * that weight: the norm behind a sublayer, the add and the norm before the next in one
//   rotate_heads    a run of heads of a row turned in pairs by the token's angles and scaled, in place
//   add_rows        hidden += delta (+ other rows) (+ one vector for all rows)
//   assemble_heads  queries, keys and values of a projected row normed, turned, blended and widened to one head width
//   scale_heads     every head of a row times the squashed gate of that head
//   soft_cap        cap * tanh(x / cap)
// Norm statistics, cosines and sines, blends and gates are float32 in every run dtype.
#include "common.h"

__device__ __forceinline__ void store_four(float* dst, float a, float b, float c, float d) {
  *(float4*)dst = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store_four(bf16_t* dst, float a, float b, float c, float d) {
  typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
  *(bf16x4*)dst = (bf16x4){(bf16_t)a, (bf16_t)b, (bf16_t)c, (bf16_t)d};
}

// ---------------------------------------------------------------------------- the stream in the run dtype
__global__ __launch_bounds__(256) void stream_rows_kernel(float* __restrict__ hidden, const float* __restrict__ delta, int parts,
                                                          size_t part_stride, bf16_t* __restrict__ out, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float v = hidden[i];
  if (delta) {
    for (int p = 0; p < parts; ++p) v += delta[p * part_stride + i];
    hidden[i] = v;
  }
  if (out) out[i] = (bf16_t)v;
}

// `out` null: a float32 run, whose sublayers read the stream itself
extern "C" int llmserve_stream_rows(float* hidden, const float* delta, int parts, void* out, int rows, int width, hipStream_t stream) {
  if (rows <= 0 || (!delta && !out)) return 0;
  if (delta && parts < 1) return ERR_BAD_ARGUMENT;
  const size_t count = (size_t)rows * width;
  hipLaunchKernelGGL(stream_rows_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, hidden, delta, parts, count,
                     (bf16_t*)out, count);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- norm of a result, added to the stream
// hidden[t] += u * rsqrt(mean(u^2) + eps) * weight with u = update[0][t] + update[1][t] + ... (the parts of a product
// cut over K, added in order).  One block per row; a row whose length is a multiple of 4 stays in registers in
// 16-byte pieces, and all of a thread's loads are asked for before the first is used.  The sum of squares is added
// in an order that depends only on the row length.  `out` (run dtype) gets the new row, or is null.
template <int PARTS, int PIECES>
__device__ __forceinline__ void add_parts(float4 (&v)[PIECES], const float* from, size_t part_stride, int quads) {
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = min((int)(threadIdx.x + j * blockDim.x), quads - 1);
    float4 d[PARTS];
#pragma unroll
    for (int p = 0; p < PARTS; ++p) d[p] = ((const float4*)(from + (size_t)p * part_stride))[i];
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      v[j].x += d[p].x; v[j].y += d[p].y; v[j].z += d[p].z; v[j].w += d[p].w;
    }
  }
}

template <int PIECES>
__device__ __forceinline__ void add_some_parts(float4 (&v)[PIECES], const float* from, int count, size_t part_stride, int quads) {
  switch (count) {
    case 1: add_parts<1, PIECES>(v, from, part_stride, quads); break;
    case 2: add_parts<2, PIECES>(v, from, part_stride, quads); break;
    case 3: add_parts<3, PIECES>(v, from, part_stride, quads); break;
    case 4: add_parts<4, PIECES>(v, from, part_stride, quads); break;
    case 5: add_parts<5, PIECES>(v, from, part_stride, quads); break;
    case 6: add_parts<6, PIECES>(v, from, part_stride, quads); break;
    default: add_parts<7, PIECES>(v, from, part_stride, quads); break;
  }
}

template <typename TO, int PIECES>
__global__ __launch_bounds__(1024) void add_normed_vector_kernel(float* __restrict__ hidden, const float* __restrict__ update,
                                                                 int parts, size_t part_stride, const void* __restrict__ weight,
                                                                 int weight_is_float, TO* __restrict__ out, int width, float eps,
                                                                 const void* __restrict__ next_weight, int next_is_float,
                                                                 float next_eps) {
  __shared__ float shared[17];
  const int quads = width / 4;
  float4* row = (float4*)(hidden + (size_t)blockIdx.x * width);
  const float* from = update + (size_t)blockIdx.x * width;
  float4 h[PIECES], u[PIECES], wide[PIECES];
  uint2 narrow[PIECES];
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = min((int)(threadIdx.x + j * blockDim.x), quads - 1);
    h[j] = row[i];
    u[j] = ((const float4*)from)[i];
    if (weight_is_float)
      wide[j] = ((const float4*)weight)[i];
    else
      narrow[j] = ((const uint2*)weight)[i];
  }
  // the further parts are added in order, up to seven at a time: their loads are all asked for before the first is used
  for (int first = 1; first < parts; first += 7)
    add_some_parts<PIECES>(u, from + (size_t)first * part_stride, min(parts - first, 7), part_stride, quads);
  float squares = 0.f;
#pragma unroll
  for (int j = 0; j < PIECES; ++j)
    if ((int)(threadIdx.x + j * blockDim.x) < quads) squares += u[j].x * u[j].x + u[j].y * u[j].y + u[j].z * u[j].z + u[j].w * u[j].w;
  const float scale = rsqrtf(block_sum(squares, shared) / (float)width + eps);
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i < quads) {
      float4 w = wide[j];
      if (!weight_is_float)  // a bfloat16 is the upper half of the float32 of the same value
        w = make_float4(__uint_as_float(narrow[j].x << 16), __uint_as_float(narrow[j].x & 0xffff0000u),
                        __uint_as_float(narrow[j].y << 16), __uint_as_float(narrow[j].y & 0xffff0000u));
      const float4 r = make_float4(h[j].x + u[j].x * scale * w.x, h[j].y + u[j].y * scale * w.y, h[j].z + u[j].z * scale * w.z,
                                   h[j].w + u[j].w * scale * w.w);
      row[i] = r;
      h[j] = r;
      if (out && !next_weight) store_four(out + (size_t)blockIdx.x * width + 4 * i, r.x, r.y, r.z, r.w);
    }
  }
  if (!next_weight) return;  // (the same for the whole block)
  // the norm before the next sublayer, of the row as it now is: its weight is asked for ahead of the block's sum
  float4 next[PIECES];
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = min((int)(threadIdx.x + j * blockDim.x), quads - 1);
    if (next_is_float) {
      next[j] = ((const float4*)next_weight)[i];
    } else {
      const uint2 raw = ((const uint2*)next_weight)[i];
      next[j] = make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                            __uint_as_float(raw.y & 0xffff0000u));
    }
  }
  float again = 0.f;
#pragma unroll
  for (int j = 0; j < PIECES; ++j)
    if ((int)(threadIdx.x + j * blockDim.x) < quads) again += h[j].x * h[j].x + h[j].y * h[j].y + h[j].z * h[j].z + h[j].w * h[j].w;
  const float next_scale = rsqrtf(block_sum(again, shared) / (float)width + next_eps);
#pragma unroll
  for (int j = 0; j < PIECES; ++j) {
    const int i = threadIdx.x + j * blockDim.x;
    if (i < quads)
      store_four(out + (size_t)blockIdx.x * width + 4 * i, h[j].x * next_scale * next[j].x, h[j].y * next_scale * next[j].y,
                 h[j].z * next_scale * next[j].z, h[j].w * next_scale * next[j].w);
  }
}

template <typename TO>
__global__ __launch_bounds__(256) void add_normed_kernel(float* __restrict__ hidden, const float* __restrict__ update, int parts,
                                                         size_t part_stride, const void* __restrict__ weight, int weight_is_float,
                                                         TO* __restrict__ out, int width, float eps,
                                                         const void* __restrict__ next_weight, int next_is_float, float next_eps) {
  __shared__ float shared[17];
  float* row = hidden + (size_t)blockIdx.x * width;
  const float* from = update + (size_t)blockIdx.x * width;
  float squares = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float u = from[i];
    for (int p = 1; p < parts; ++p) u += from[p * part_stride + i];
    squares += u * u;
  }
  const float scale = rsqrtf(block_sum(squares, shared) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float u = from[i];
    for (int p = 1; p < parts; ++p) u += from[p * part_stride + i];
    const float r = row[i] + u * scale * load_as_float(weight, weight_is_float, i);
    row[i] = r;
    if (out && !next_weight) out[(size_t)blockIdx.x * width + i] = from_float<TO>(r);
  }
  if (!next_weight) return;
  float again = 0.f;  // (a thread reads back what it wrote itself)
  for (int i = threadIdx.x; i < width; i += blockDim.x) again += row[i] * row[i];
  const float next_scale = rsqrtf(block_sum(again, shared) / (float)width + next_eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x)
    out[(size_t)blockIdx.x * width + i] = from_float<TO>(row[i] * next_scale * load_as_float(next_weight, next_is_float, i));
}

template <typename TO>
static void launch_add_normed(float* hidden, const float* update, int parts, const void* weight, int weight_is_float, TO* out,
                              int rows, int width, float eps, hipStream_t stream, const void* next_weight = nullptr,
                              int next_is_float = 0, float next_eps = 0.f) {
  const size_t part_stride = (size_t)rows * width;
  if (width % 4 == 0 && width <= 1024 * 4 * 4) {
    const int quads = width / 4;
    const int pieces = quads <= 1024 ? 1 : quads <= 2048 ? 2 : 4;
    const int threads = ((quads + pieces - 1) / pieces + WAVE - 1) / WAVE * WAVE;
    if (pieces == 1)
      hipLaunchKernelGGL((add_normed_vector_kernel<TO, 1>), dim3(rows), dim3(threads), 0, stream, hidden, update, parts, part_stride,
                         weight, weight_is_float, out, width, eps, next_weight, next_is_float, next_eps);
    else if (pieces == 2)
      hipLaunchKernelGGL((add_normed_vector_kernel<TO, 2>), dim3(rows), dim3(threads), 0, stream, hidden, update, parts, part_stride,
                         weight, weight_is_float, out, width, eps, next_weight, next_is_float, next_eps);
    else
      hipLaunchKernelGGL((add_normed_vector_kernel<TO, 4>), dim3(rows), dim3(threads), 0, stream, hidden, update, parts, part_stride,
                         weight, weight_is_float, out, width, eps, next_weight, next_is_float, next_eps);
    return;
  }
  hipLaunchKernelGGL(add_normed_kernel<TO>, dim3(rows), dim3(256), 0, stream, hidden, update, parts, part_stride, weight,
                     weight_is_float, out, width, eps, next_weight, next_is_float, next_eps);
}

// `out` null, or bfloat16 rows (out_is_float 0), or float32 rows
extern "C" int llmserve_add_normed(float* hidden, const float* update, int parts, const void* weight, int weight_is_float, void* out,
                                   int out_is_float, int rows, int width, float eps, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (!update || parts < 1 || width < 1) return ERR_BAD_ARGUMENT;
  if (out_is_float)
    launch_add_normed<float>(hidden, update, parts, weight, weight_is_float, (float*)out, rows, width, eps, stream);
  else
    launch_add_normed<bf16_t>(hidden, update, parts, weight, weight_is_float, (bf16_t*)out, rows, width, eps, stream);
  return LAUNCH_STATUS();
}

// The same, and then the norm before the next sublayer: out = new row * rsqrt(mean(new row^2) + next_eps) * next_weight.
extern "C" int llmserve_add_normed_norm(float* hidden, const float* update, int parts, const void* weight, int weight_is_float,
                                        float eps, const void* next_weight, int next_is_float, float next_eps, void* out,
                                        int out_is_float, int rows, int width, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (!update || !next_weight || !out || parts < 1 || width < 1) return ERR_BAD_ARGUMENT;
  if (out_is_float)
    launch_add_normed<float>(hidden, update, parts, weight, weight_is_float, (float*)out, rows, width, eps, stream, next_weight,
                             next_is_float, next_eps);
  else
    launch_add_normed<bf16_t>(hidden, update, parts, weight, weight_is_float, (bf16_t*)out, rows, width, eps, stream, next_weight,
                              next_is_float, next_eps);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- heads turned in place
// For every token and every one of `heads` heads (`head_stride` columns each, from column `first` of a row `x_width`
// wide): the first `dims` columns turn in pairs (pairing 1: (2i, 2i + 1); 2: (i, i + dims / 2)) by (cos, sin) of
// table[token][i], and every column of a head from head `scale_from` on is multiplied by `scale` (queries and keys side by
// side are one launch, the keys scaled).  float32 arithmetic; a thread a pair, or a column beyond the pairs.
template <typename T>
__global__ __launch_bounds__(256) void rotate_heads_kernel(T* __restrict__ x, int x_width, int first, int head_stride, int heads,
                                                           const float* __restrict__ table, int dims, int pairing, float later_scale,
                                                           int scale_from) {
  const size_t token = blockIdx.x;
  T* row = x + token * x_width + first;
  const int half = dims / 2, per_head = head_stride - half;  // work items a head: the pairs, then the columns left
  for (int item = threadIdx.x; item < heads * per_head; item += blockDim.x) {
    const int head = item / per_head, inside = item - head * per_head;
    T* at = row + (size_t)head * head_stride;
    const float scale = head >= scale_from ? later_scale : 1.f;
    if (inside < half) {
      const int a_at = pairing == 1 ? 2 * inside : inside, b_at = pairing == 1 ? 2 * inside + 1 : inside + half;
      const float2 cs = ((const float2*)table)[token * half + inside];
      const float a = to_float(at[a_at]), b = to_float(at[b_at]);
      at[a_at] = from_float<T>((a * cs.x - b * cs.y) * scale);
      at[b_at] = from_float<T>((b * cs.x + a * cs.y) * scale);
    } else if (scale != 1.f) {
      const int column = dims + inside - half;
      at[column] = from_float<T>(to_float(at[column]) * scale);
    }
  }
}

extern "C" int llmserve_rotate_heads(void* x, int is_float, int tokens, int x_width, int first, int head_stride, int heads,
                                     const float* table, int dims, int pairing, float scale, int scale_from, hipStream_t stream) {
  if (tokens <= 0 || heads <= 0) return 0;
  if (dims < 0 || dims % 2 || dims > head_stride || first < 0 || first + heads * head_stride > x_width || (dims > 0 && !table) ||
      (dims > 0 && pairing != 1 && pairing != 2))
    return ERR_BAD_ARGUMENT;
  if (is_float)
    hipLaunchKernelGGL(rotate_heads_kernel<float>, dim3(tokens), dim3(256), 0, stream, (float*)x, x_width, first, head_stride, heads,
                       table, dims, pairing, scale, scale_from);
  else
    hipLaunchKernelGGL(rotate_heads_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream, (bf16_t*)x, x_width, first, head_stride, heads,
                       table, dims, pairing, scale, scale_from);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- rows and a vector added to the stream
// hidden[t] += delta[0][t] + delta[1][t] + ... (+ other[t]) (+ vector), float32, in place; any of the three may be null.
__global__ __launch_bounds__(256) void add_rows_kernel(float* __restrict__ hidden, const float* __restrict__ delta, int parts,
                                                       size_t part_stride, const float* __restrict__ other,
                                                       const float* __restrict__ vector, int width, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float v = hidden[i];
  if (delta)
    for (int p = 0; p < parts; ++p) v += delta[p * part_stride + i];
  if (other) v += other[i];
  if (vector) v += vector[i % width];
  hidden[i] = v;
}

extern "C" int llmserve_add_rows(float* hidden, const float* delta, int parts, const float* other, const float* vector, int rows,
                                 int width, hipStream_t stream) {
  if (rows <= 0 || (!delta && !other && !vector)) return 0;
  if (delta && parts < 1) return ERR_BAD_ARGUMENT;
  const size_t count = (size_t)rows * width;
  hipLaunchKernelGGL(add_rows_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, hidden, delta, parts, count, other,
                     vector, width, count);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- heads put together for the attention
// One block per token, a wave a head at a time.  A query or key head of `dim` is RMS-normed (norm 1: by itself, the
// weight of `dim` shared by the heads; 2: all heads of the projection together, the weight as long as they; 0: not),
// its first `rot_dims` dimensions are turned in pairs (2i, 2i + 1), or with `pairing` 2 in pairs (i, i + rot_dims / 2), by
// (cos, sin) of table[token][i], and it is written
// `width` wide, zeros beyond `dim`.  A value head of `vdim` is blended with the same columns of `other` and written
// `width` wide.  The output row is [heads | kv_heads | kv_heads] heads of `width`; the keys and values may go to
// their pages in the same kernel (a step of single tokens: one launch less).
struct HeadSizes {
  int x_width, q_first, k_first, v_first, heads, kv_heads, dim, vdim, width, norm, rot_dims, other_width, other_first, pairing;
};

template <typename T>
__global__ __launch_bounds__(1024) void assemble_heads_kernel(const T* __restrict__ x, HeadSizes z, const void* __restrict__ q_weight,
                                                              const void* __restrict__ k_weight, int weight_is_float, float eps,
                                                              const float* __restrict__ table, const T* __restrict__ other,
                                                              float blend, T* __restrict__ out, T* __restrict__ keys,
                                                              T* __restrict__ values, const int* __restrict__ slots, int page_size) {
  __shared__ float shared[17];
  const size_t token = blockIdx.x;
  const T* row = x + token * z.x_width;
  T* dst = out + token * (size_t)(z.heads + 2 * z.kv_heads) * z.width;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = blockDim.x >> 6;
  float q_scale = 1.f, k_scale = 1.f;
  if (z.norm == 2) {
    float squares = 0.f;
    for (int e = threadIdx.x; e < z.heads * z.dim; e += blockDim.x) {
      const float v = to_float(row[z.q_first + e]);
      squares += v * v;
    }
    q_scale = rsqrtf(block_sum(squares, shared) / (float)(z.heads * z.dim) + eps);
    squares = 0.f;
    for (int e = threadIdx.x; e < z.kv_heads * z.dim; e += blockDim.x) {
      const float v = to_float(row[z.k_first + e]);
      squares += v * v;
    }
    k_scale = rsqrtf(block_sum(squares, shared) / (float)(z.kv_heads * z.dim) + eps);
  }
  const float* angles = table ? table + token * z.rot_dims : nullptr;  // rot_dims / 2 pairs of (cos, sin)
  for (int unit = wave; unit < z.heads + z.kv_heads; unit += waves) {
    const bool is_key = unit >= z.heads;
    const int head = is_key ? unit - z.heads : unit;
    const T* src = row + (is_key ? z.k_first : z.q_first) + head * z.dim;
    const void* weight = is_key ? k_weight : q_weight;
    const int weight_first = z.norm == 2 ? head * z.dim : 0;
    float scale = is_key ? k_scale : q_scale;
    if (z.norm == 1) {
      float squares = 0.f;
      for (int e = lane; e < z.dim; e += WAVE) {
        const float v = to_float(src[e]);
        squares += v * v;
      }
      scale = rsqrtf(wave_sum(squares) / (float)z.dim + eps);
    }
    for (int e = lane; e < z.width; e += WAVE) {
      float result = 0.f;
      if (e < z.dim) {
        float mine = to_float(src[e]) * scale;
        if (z.norm) mine *= load_as_float(weight, weight_is_float, weight_first + e);
        result = mine;
        if (e < z.rot_dims) {
          const int half = z.rot_dims / 2;
          const int other_e = z.pairing == 2 ? (e < half ? e + half : e - half) : (e ^ 1);
          const int pair = z.pairing == 2 ? (e < half ? e : e - half) : (e >> 1);
          const bool second = z.pairing == 2 ? e >= half : (e & 1);
          float partner = to_float(src[other_e]) * scale;
          if (z.norm) partner *= load_as_float(weight, weight_is_float, weight_first + other_e);
          const float c = angles[2 * pair], s = angles[2 * pair + 1];
          result = second ? mine * c + partner * s : mine * c - partner * s;
        }
      }
      dst[(size_t)unit * z.width + e] = from_float<T>(result);
    }
  }
  const T* own = row + z.v_first;
  const T* given = other ? other + token * z.other_width + z.other_first : nullptr;
  T* value_dst = dst + (size_t)(z.heads + z.kv_heads) * z.width;
  for (int index = threadIdx.x; index < z.kv_heads * z.width; index += blockDim.x) {
    const int head = index / z.width, e = index % z.width;
    float result = 0.f;
    if (e < z.vdim) {
      result = to_float(own[head * z.vdim + e]);
      if (given) result = (1.f - blend) * result + blend * to_float(given[head * z.vdim + e]);
    }
    value_dst[index] = from_float<T>(result);
  }
  // With `slots` (page * page_size + offset of every token, negative: nowhere) the token's keys and values also go
  // to its place in the pages, read back from the row just written.
  if (slots == nullptr) return;
  const int slot = slots[token];
  if (slot < 0) return;
  __syncthreads();
  const int page = slot / page_size, offset = slot % page_size;
  const T* k_row = dst + (size_t)z.heads * z.width;
  const T* v_row = k_row + (size_t)z.kv_heads * z.width;
  for (int index = threadIdx.x; index < z.kv_heads * z.width; index += blockDim.x) {
    const int head = index / z.width, d = index % z.width;
    const size_t block = ((size_t)page * z.kv_heads + head) * page_size * z.width;
    keys[block + key_element(d, offset, page_size, z.width)] = k_row[index];
    values[block + value_element(d, offset, page_size, z.width)] = v_row[index];
  }
}

extern "C" int llmserve_assemble_heads(const void* x, int is_float, int tokens, int x_width, int q_first, int k_first, int v_first,
                                       int heads, int kv_heads, int dim, int vdim, int width, int norm, const void* q_weight,
                                       const void* k_weight, int weight_is_float, float eps, const float* table, int rot_dims,
                                       const void* other, int other_width, int other_first, float blend, void* out,
                                       void* keys, void* values, const int* slots, int page_size, int pairing, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (pairing < 1 || pairing > 2) return ERR_BAD_ARGUMENT;
  if (heads < 1 || kv_heads < 1 || dim < 1 || vdim < 1 || width < dim || width < vdim || norm < 0 || norm > 2 ||
      (norm && (!q_weight || !k_weight)) || rot_dims < 0 || rot_dims % 2 || rot_dims > dim || (rot_dims && !table) ||
      q_first < 0 || k_first < 0 || v_first < 0 || q_first + heads * dim > x_width || k_first + kv_heads * dim > x_width ||
      v_first + kv_heads * vdim > x_width || (other && (other_first < 0 || other_first + kv_heads * vdim > other_width)))
    return ERR_BAD_ARGUMENT;
  const HeadSizes z = {x_width, q_first, k_first, v_first, heads, kv_heads, dim, vdim, width, norm, rot_dims, other_width, other_first, pairing};
  if (slots && (!keys || !values || page_size < 1)) return ERR_BAD_ARGUMENT;
  // a wave a head where there are up to sixteen of them (a step of few tokens is as long as its longest workgroup)
  const int threads = WAVE * max(4, min(16, heads + kv_heads));
  if (is_float)
    hipLaunchKernelGGL(assemble_heads_kernel<float>, dim3(tokens), dim3(threads), 0, stream, (const float*)x, z, q_weight, k_weight,
                       weight_is_float, eps, table, (const float*)other, blend, (float*)out, (float*)keys, (float*)values, slots,
                       page_size);
  else
    hipLaunchKernelGGL(assemble_heads_kernel<bf16_t>, dim3(tokens), dim3(threads), 0, stream, (const bf16_t*)x, z, q_weight, k_weight,
                       weight_is_float, eps, table, (const bf16_t*)other, blend, (bf16_t*)out, (bf16_t*)keys, (bf16_t*)values, slots,
                       page_size);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- a gate a head
template <typename T>
__global__ __launch_bounds__(256) void scale_heads_kernel(T* __restrict__ x, int heads, int width, const T* __restrict__ gates,
                                                          int gate_stride, int gate_first, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const size_t token = i / ((size_t)heads * width);
  const int head = (int)((i / width) % heads);
  const float gate = to_float(gates[token * gate_stride + gate_first + head]);
  x[i] = from_float<T>(to_float(x[i]) / (1.f + expf(-gate)));
}

extern "C" int llmserve_scale_heads(void* x, int is_float, int tokens, int heads, int width, const void* gates, int gate_stride,
                                    int gate_first, hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (heads < 1 || width < 1 || gate_first < 0 || gate_first + heads > gate_stride) return ERR_BAD_ARGUMENT;
  const size_t count = (size_t)tokens * heads * width;
  const dim3 grid((unsigned)((count + 255) / 256));
  if (is_float)
    hipLaunchKernelGGL(scale_heads_kernel<float>, grid, dim3(256), 0, stream, (float*)x, heads, width, (const float*)gates, gate_stride,
                       gate_first, count);
  else
    hipLaunchKernelGGL(scale_heads_kernel<bf16_t>, grid, dim3(256), 0, stream, (bf16_t*)x, heads, width, (const bf16_t*)gates,
                       gate_stride, gate_first, count);
  return LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------- capped values
__global__ __launch_bounds__(256) void soft_cap_kernel(float* __restrict__ x, float cap, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int llmserve_soft_cap(float* x, int rows, int width, float cap, hipStream_t stream) {
  if (rows <= 0 || width <= 0) return 0;
  if (!(cap > 0.f)) return ERR_BAD_ARGUMENT;
  const size_t count = (size_t)rows * width;
  hipLaunchKernelGGL(soft_cap_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, x, cap, count);
  return LAUNCH_STATUS();
}
