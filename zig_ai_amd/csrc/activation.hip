// SwiGLU gate on the fused gate|up projection:
//   out[t, i] = silu(gu[t, i]) * gu[t, I + i],   silu(g) = g / (1 + exp(-g))
// computed in 32-bit (/root/reference/src/transformer/ffn.zig:24-30,
// /root/reference/src/cuda/layer_kernels.cu:62-70).
// Also the element-wise cast between storage types.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens, int inter) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)n_tokens * inter;
  if (idx >= total) return;
  const size_t t = idx / inter, i = idx % inter;
  const float g = to_f32<T>(gu[t * 2 * inter + i]);
  const float u = to_f32<T>(gu[t * 2 * inter + inter + i]);
  const float sig = 1.0f / (1.0f + expf(-g));
  out[idx] = from_f32<T>(g * sig * u);
}

template <typename T>
__global__ void __launch_bounds__(256)
swiglu_vec8_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens, int inter) {
  const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  const size_t total = (size_t)n_tokens * inter;
  if (idx >= total) return;
  const size_t t = idx / inter, i = idx % inter;
  float g[8], u[8], o[8];
  load8<T>(gu + t * 2 * inter + i, g);
  load8<T>(gu + t * 2 * inter + inter + i, u);
#pragma unroll
  for (int k = 0; k < 8; ++k) o[k] = g[k] * (1.0f / (1.0f + expf(-g[k]))) * u[k];
  store8<T>(out + idx, o);
}

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < n) out[idx] = from_f32<TO>(to_f32<TI>(in[idx]));
}

extern "C" int za_swiglu(const void* gu, void* out, int dtype, int n_tokens, int inter,
                         hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || inter <= 0 || !gu || !out) return ZA_ERR_ARG;
  const size_t total = (size_t)n_tokens * inter;
  const bool vec = inter % 8 == 0;
  const size_t threads = vec ? total / 8 : total;
  dim3 grid((unsigned)((threads + 255) / 256)), block(256);
  if (dtype == 0) {
    if (vec)
      hipLaunchKernelGGL((swiglu_vec8_kernel<float>), grid, block, 0, stream, (const float*)gu,
                         (float*)out, n_tokens, inter);
    else
      hipLaunchKernelGGL((swiglu_kernel<float>), grid, block, 0, stream, (const float*)gu,
                         (float*)out, n_tokens, inter);
  } else if (dtype == 1) {
    if (vec)
      hipLaunchKernelGGL((swiglu_vec8_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)gu,
                         (bf16_t*)out, n_tokens, inter);
    else
      hipLaunchKernelGGL((swiglu_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)gu,
                         (bf16_t*)out, n_tokens, inter);
  } else {
    return ZA_ERR_UNSUPPORTED;
  }
  return za_launch_status();
}

// dtype codes: 0 = float32, 1 = bfloat16
extern "C" int za_cast(const void* in, int in_dtype, void* out, int out_dtype, long long n,
                       hipStream_t stream) {
  if (n == 0) return 0;
  if (n < 0 || !in || !out) return ZA_ERR_ARG;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (in_dtype == 0 && out_dtype == 1)
    hipLaunchKernelGGL((cast_kernel<float, bf16_t>), grid, block, 0, stream, (const float*)in,
                       (bf16_t*)out, (size_t)n);
  else if (in_dtype == 1 && out_dtype == 0)
    hipLaunchKernelGGL((cast_kernel<bf16_t, float>), grid, block, 0, stream, (const bf16_t*)in,
                       (float*)out, (size_t)n);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}

// Columns [col0, col0 + ncols) of every row of `in` [rows, in_width] into columns
// [out_col0, out_col0 + ncols) of `out` [rows, out_width], converted between the two
// storage types: how a mixer takes q, k and v out of a fused projection's rows and puts
// them back side by side, without the tensor library.
template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
copy_columns_kernel(const TI* __restrict__ in, TO* __restrict__ out, int in_width, int col0,
                    int out_width, int out_col0, int ncols, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t row = idx / ncols;
  const int c = (int)(idx % ncols);
  out[row * out_width + out_col0 + c] = from_f32<TO>(to_f32<TI>(in[row * in_width + col0 + c]));
}

extern "C" int za_copy_columns(const void* in, int in_dtype, int in_width, int col0, void* out,
                               int out_dtype, int out_width, int out_col0, int rows, int ncols,
                               hipStream_t stream) {
  if (rows == 0 || ncols == 0) return 0;
  if (rows < 0 || ncols < 0 || !in || !out || col0 < 0 || out_col0 < 0 ||
      col0 + ncols > in_width || out_col0 + ncols > out_width)
    return ZA_ERR_ARG;
  const size_t total = (size_t)rows * ncols;
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
#define ZA_COPY_COLUMNS(TI, TO)                                                                   \
  hipLaunchKernelGGL((copy_columns_kernel<TI, TO>), grid, block, 0, stream, (const TI*)in, (TO*)out, \
                     in_width, col0, out_width, out_col0, ncols, total)
  if (in_dtype == 0 && out_dtype == 0) ZA_COPY_COLUMNS(float, float);
  else if (in_dtype == 0 && out_dtype == 1) ZA_COPY_COLUMNS(float, bf16_t);
  else if (in_dtype == 1 && out_dtype == 0) ZA_COPY_COLUMNS(bf16_t, float);
  else if (in_dtype == 1 && out_dtype == 1) ZA_COPY_COLUMNS(bf16_t, bf16_t);
  else return ZA_ERR_UNSUPPORTED;
#undef ZA_COPY_COLUMNS
  return za_launch_status();
}

// A gated linear unit with bounded inputs, on the fused gate|up projection:
//   g = min(gu[t, i], limit);  u = clamp(gu[t, I + i], -limit, limit)
//   out[t, i] = g * sigmoid(alpha * g) * (u + up_offset)
// in 32-bit.  `limit <= 0` means no bound.
template <typename T>
__global__ void __launch_bounds__(256)
clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens, int inter,
                   float limit, float alpha, float up_offset) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)n_tokens * inter;
  if (idx >= total) return;
  const size_t t = idx / inter, i = idx % inter;
  float g = to_f32<T>(gu[t * 2 * inter + i]);
  float u = to_f32<T>(gu[t * 2 * inter + inter + i]);
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  out[idx] = from_f32<T>(g * (1.0f / (1.0f + expf(-alpha * g))) * (u + up_offset));
}

template <typename T>
__global__ void __launch_bounds__(256)
clamped_glu_vec8_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens, int inter,
                        float limit, float alpha, float up_offset) {
  const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  const size_t total = (size_t)n_tokens * inter;
  if (idx >= total) return;
  const size_t t = idx / inter, i = idx % inter;
  float g[8], u[8], o[8];
  load8<T>(gu + t * 2 * inter + i, g);
  load8<T>(gu + t * 2 * inter + inter + i, u);
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float gk = g[k], uk = u[k];
    if (limit > 0.f) {
      gk = fminf(gk, limit);
      uk = fminf(fmaxf(uk, -limit), limit);
    }
    o[k] = gk * (1.0f / (1.0f + expf(-alpha * gk))) * (uk + up_offset);
  }
  store8<T>(out + idx, o);
}

extern "C" int za_clamped_glu(const void* gu, void* out, int dtype, int n_tokens, int inter,
                              float limit, float alpha, float up_offset, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || inter <= 0 || !gu || !out) return ZA_ERR_ARG;
  const size_t total = (size_t)n_tokens * inter;
  const bool vec = inter % 8 == 0;      // rows of both halves start on 16-byte boundaries
  const size_t threads = vec ? total / 8 : total;
  dim3 grid((unsigned)((threads + 255) / 256)), block(256);
#define ZA_GLU(KERNEL, T)                                                                      \
  hipLaunchKernelGGL((KERNEL<T>), grid, block, 0, stream, (const T*)gu, (T*)out, n_tokens, inter, \
                     limit, alpha, up_offset)
  if (dtype == 0) {
    if (vec) ZA_GLU(clamped_glu_vec8_kernel, float); else ZA_GLU(clamped_glu_kernel, float);
  } else if (dtype == 1) {
    if (vec) ZA_GLU(clamped_glu_vec8_kernel, bf16_t); else ZA_GLU(clamped_glu_kernel, bf16_t);
  } else {
    return ZA_ERR_UNSUPPORTED;
  }
#undef ZA_GLU
  return za_launch_status();
}

// A gated unit on the fused gate|up projection with a choice of activation:
//   out[t, i] = act(gu[t, i]) * gu[t, I + i]
//   act 0: silu(g) = g / (1 + exp(-g))
//   act 1: gelu in its tanh form, 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))
// in 32-bit.
__device__ __forceinline__ float gate_act(float g, int act) {
  if (act == 1) {
    const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return 0.5f * g * (1.0f + tanhf(z));
  }
  return g * (1.0f / (1.0f + expf(-g)));
}

template <typename T, int VEC>
__global__ void __launch_bounds__(256)
gated_unit_kernel(const T* __restrict__ gu, T* __restrict__ out, int n_tokens, int inter, int act) {
  const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  const size_t total = (size_t)n_tokens * inter;
  if (idx >= total) return;
  const size_t t = idx / inter, i = idx % inter;
  if (VEC == 8) {
    float g[8], u[8], o[8];
    load8<T>(gu + t * 2 * inter + i, g);
    load8<T>(gu + t * 2 * inter + inter + i, u);
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = gate_act(g[k], act) * u[k];
    store8<T>(out + idx, o);
  } else {
    const float g = to_f32<T>(gu[t * 2 * inter + i]);
    const float u = to_f32<T>(gu[t * 2 * inter + inter + i]);
    out[idx] = from_f32<T>(gate_act(g, act) * u);
  }
}

extern "C" int za_gated_unit(const void* gu, void* out, int dtype, int n_tokens, int inter, int act,
                             hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || inter <= 0 || !gu || !out || act < 0 || act > 1) return ZA_ERR_ARG;
  const size_t total = (size_t)n_tokens * inter;
  const bool vec = inter % 8 == 0;
  const size_t threads = vec ? total / 8 : total;
  dim3 grid((unsigned)((threads + 255) / 256)), block(256);
#define ZA_UNIT(T, V)                                                                          \
  hipLaunchKernelGGL((gated_unit_kernel<T, V>), grid, block, 0, stream, (const T*)gu, (T*)out, \
                     n_tokens, inter, act)
  if (dtype == 0) {
    if (vec) ZA_UNIT(float, 8); else ZA_UNIT(float, 1);
  } else if (dtype == 1) {
    if (vec) ZA_UNIT(bf16_t, 8); else ZA_UNIT(bf16_t, 1);
  } else {
    return ZA_ERR_UNSUPPORTED;
  }
#undef ZA_UNIT
  return za_launch_status();
}

// A feed-forward's activation on its own, element by element, in 32-bit:
//   act 0: the square of relu, max(x, 0)^2
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
activate_kernel(const T* __restrict__ in, T* __restrict__ out, size_t total, int act) {
  const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (idx >= total) return;
  if (VEC == 8) {
    float x[8], o[8];
    load8<T>(in + idx, x);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float r = fmaxf(x[k], 0.f);
      o[k] = r * r;
    }
    store8<T>(out + idx, o);
  } else {
    const float r = fmaxf(to_f32<T>(in[idx]), 0.f);
    out[idx] = from_f32<T>(r * r);
  }
}

extern "C" int za_activate(const void* in, void* out, int dtype, long long n, int act,
                           hipStream_t stream) {
  if (n == 0) return 0;
  if (n < 0 || !in || !out || act != 0) return ZA_ERR_ARG;
  const size_t total = (size_t)n;
  const bool vec = total % 8 == 0;
  const size_t threads = vec ? total / 8 : total;
  dim3 grid((unsigned)((threads + 255) / 256)), block(256);
#define ZA_ACT(T, V)                                                                         \
  hipLaunchKernelGGL((activate_kernel<T, V>), grid, block, 0, stream, (const T*)in, (T*)out, \
                     total, act)
  if (dtype == 0) {
    if (vec) ZA_ACT(float, 8); else ZA_ACT(float, 1);
  } else if (dtype == 1) {
    if (vec) ZA_ACT(bf16_t, 8); else ZA_ACT(bf16_t, 1);
  } else {
    return ZA_ERR_UNSUPPORTED;
  }
#undef ZA_ACT
  return za_launch_status();
}

// out[r, c] = in[r, c] + bias[c]: the bias of a product whose 32-bit sums another kernel (or
// a library) left, rounded once into the result's type.  `out` may be `in` for 32-bit results.
template <typename TO>
__global__ void __launch_bounds__(256)
bias_add_kernel(const float* __restrict__ in, const float* __restrict__ bias, TO* __restrict__ out,
                size_t total, int N) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  out[idx] = from_f32<TO>(in[idx] + bias[idx % N]);
}

extern "C" int za_bias_add(const float* in, const float* bias, void* out, int out_dtype,
                           long long rows, int N, hipStream_t stream) {
  if (rows == 0) return 0;
  if (rows < 0 || N <= 0 || !in || !bias || !out) return ZA_ERR_ARG;
  const size_t total = (size_t)rows * N;
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (out_dtype == 0)
    hipLaunchKernelGGL((bias_add_kernel<float>), grid, block, 0, stream, in, bias, (float*)out,
                       total, N);
  else if (out_dtype == 1)
    hipLaunchKernelGGL((bias_add_kernel<bf16_t>), grid, block, 0, stream, in, bias, (bf16_t*)out,
                       total, N);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}

// x <- x * s, 32-bit, in place (an output head's constant factor on its logits).
__global__ void __launch_bounds__(256) scale_kernel(float* __restrict__ x, float s, size_t n) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < n) x[idx] *= s;
}

extern "C" int za_scale(float* x, float s, long long n, hipStream_t stream) {
  if (n == 0) return 0;
  if (n < 0 || !x) return ZA_ERR_ARG;
  hipLaunchKernelGGL(scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, s,
                     (size_t)n);
  return za_launch_status();
}

// x <- cap * tanh(x / cap), 32-bit, in place (an output head's cap on its logits).
__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ x, float cap, size_t n) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < n) x[idx] = cap * tanhf(x[idx] / cap);
}

extern "C" int za_softcap(float* x, float cap, long long n, hipStream_t stream) {
  if (n == 0) return 0;
  if (n < 0 || !x || !(cap > 0.f)) return ZA_ERR_ARG;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x,
                     cap, (size_t)n);
  return za_launch_status();
}

// out[t][j] = act(g[t][j]) * table[ids[t]][col0 + j]: a gate (computed from something
// else) on a slice of a table row that the token's id picks.  `table` has `ld` columns
// and `rows` rows; an id outside the table yields zeros.
template <typename T, typename TT>
__global__ void __launch_bounds__(256)
table_gate_kernel(const T* __restrict__ g, const int* __restrict__ ids,
                  const TT* __restrict__ table, int rows, int ld, int col0, T* __restrict__ out,
                  int n_tokens, int dim, int act) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (size_t)n_tokens * dim) return;
  const size_t t = idx / dim;
  const int j = (int)(idx % dim), id = ids[t];
  const float e = (id >= 0 && id < rows) ? to_f32<TT>(table[(size_t)id * ld + col0 + j]) : 0.f;
  out[idx] = from_f32<T>(gate_act(to_f32<T>(g[idx]), act) * e);
}

// dtype codes: 0 = float32, 1 = bfloat16 (of g and out; the table has its own)
extern "C" int za_table_gate(const void* g, int dtype, const int* ids, const void* table,
                             int table_dtype, int rows, int ld, int col0, void* out, int n_tokens,
                             int dim, int act, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || dim <= 0 || !g || !ids || !table || !out || rows <= 0 || col0 < 0 ||
      col0 + dim > ld || act < 0 || act > 1)
    return ZA_ERR_ARG;
  dim3 grid((unsigned)(((size_t)n_tokens * dim + 255) / 256)), block(256);
#define ZA_TG(T, TT)                                                                            \
  hipLaunchKernelGGL((table_gate_kernel<T, TT>), grid, block, 0, stream, (const T*)g, ids,      \
                     (const TT*)table, rows, ld, col0, (T*)out, n_tokens, dim, act)
  if (dtype == 0 && table_dtype == 0) ZA_TG(float, float);
  else if (dtype == 0 && table_dtype == 1) ZA_TG(float, bf16_t);
  else if (dtype == 1 && table_dtype == 1) ZA_TG(bf16_t, bf16_t);
  else if (dtype == 1 && table_dtype == 0) ZA_TG(bf16_t, float);
  else return ZA_ERR_UNSUPPORTED;
#undef ZA_TG
  return za_launch_status();
}
