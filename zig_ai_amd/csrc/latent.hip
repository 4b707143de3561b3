// Attention over one small latent vector a token ("latent attention"): what is cached for
// a token is a normed latent c [R] and, optionally, a rotated key part k_r [Dr] that all
// heads share; every head's keys and values are linear expansions of c,
//     k_h = Wuk_h c,   v_h = Wuv_h c.
// Neither is ever formed.  With q_h = [q_n | q_r] (unrotated | rotated),
//     q_h . [k_h | k_r] = (Wuk_h^T q_n) . c + q_r . k_r
//     sum_j p_j v_h,j   = Wuv_h (sum_j p_j c_j)
// so the attention runs with ONE key/value head whose key is the cached row [c | k_r]
// (W = R + Dr elements) and whose value is the row's first R elements, with queries
// [Wuk_h^T q_n | q_r] and results that the head's Wuv expands afterwards.  The cache holds
// one plane of W elements a token, rows of a page one after the other.
//
// Kernels:
//   latent_prepare     a token's opening projection -> the normed query latent, and the row
//                      [rmsnorm(c) | rotate(k_r)] into the token's place in the cache
//   rotate_part        the rotated part of every head's query into the folded query
//   head_linear        out[t][h] = x[t][h] @ W[h]^T for every head at once (the two
//                      foldings above), optionally times sigmoid(gate) a head or an element
//   latent_attention   the attention itself: causal, streaming softmax in 32-bit with a sink
//                      a head, any mix of prompt portions and single tokens in one launch,
//                      contexts optionally cut into ranges (latent_combine merges them)
//   latent_attention_mfma   the same on the matrix cores (bfloat16, 16-byte pieces): four waves
//                      of 16 rows each for prompt portions and mixed steps
//   latent_decode_mfma      steps that only decode: four waves share 16 rows
// Rotation: adjacent pairs (2i, 2i + 1) or halves (i, i + dims/2) of the first `rot_dims`
// elements, angle = position * inv_freq[i] in 32-bit.
#include <math.h>

#include "common.h"

// ------------------------------------------------------------------ latent_prepare
// down: [T][ld], columns [q_col, q_col + Rq) the query latent, [c_col, c_col + R) the
// latent, then Dr elements of the rotated key part.  cq: [T][Rq].  plane: the cache,
// token t's row at plane + (slots[t] / page_size) * page_stride + (slots[t] % page_size) * W.
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const T* __restrict__ down, int ld, int q_col, int Rq, int c_col, int R,
                      int Dr, const float* __restrict__ q_norm_w, const float* __restrict__ c_norm_w,
                      float eps, const int* __restrict__ positions, const int* __restrict__ slots,
                      const float* __restrict__ inv_freq, int rot_dims, int adjacent,
                      T* __restrict__ cq, T* __restrict__ plane, int page_size,
                      long long page_stride) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const T* row = down + t * ld;
  const int tid = threadIdx.x, bd = blockDim.x;
  if (cq) {
    float ss = 0.f;
    for (int i = tid; i < Rq; i += bd) {
      const float v = to_f32<T>(row[q_col + i]);
      ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float f = 1.0f / sqrtf(ss / (float)Rq + eps);
    for (int i = tid; i < Rq; i += bd)
      cq[t * Rq + i] = from_f32<T>(to_f32<T>(row[q_col + i]) * f * q_norm_w[i]);
  }
  if (!plane) return;
  const int slot = slots[t];
  if (slot < 0) return;
  T* dst = plane + (size_t)(slot / page_size) * page_stride + (size_t)(slot % page_size) * (R + Dr);
  float ss = 0.f;
  for (int i = tid; i < R; i += bd) {
    const float v = to_f32<T>(row[c_col + i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float f = 1.0f / sqrtf(ss / (float)R + eps);
  for (int i = tid; i < R; i += bd)
    dst[i] = from_f32<T>(to_f32<T>(row[c_col + i]) * f * c_norm_w[i]);
  const T* kr = row + c_col + R;
  const int half = rot_dims / 2;
  const float pos = (float)positions[t];
  for (int i = tid; i < half; i += bd) {
    const int a = adjacent ? 2 * i : i, b = adjacent ? 2 * i + 1 : i + half;
    float sn, cs;
    sincosf(pos * inv_freq[i], &sn, &cs);
    const float u = to_f32<T>(kr[a]), v = to_f32<T>(kr[b]);
    dst[R + a] = from_f32<T>(u * cs - v * sn);
    dst[R + b] = from_f32<T>(v * cs + u * sn);
  }
  for (int i = rot_dims + tid; i < Dr; i += bd) dst[R + i] = kr[i];
}

extern "C" int za_latent_prepare(const void* down, int dtype, int ld, int q_col, int q_rank,
                                 int c_col, int kv_rank, int rot_dim, const float* q_norm_w,
                                 const float* c_norm_w, float eps, const int* positions,
                                 const int* slots, const float* inv_freq, int rot_dims,
                                 int adjacent, void* cq, void* plane, int page_size,
                                 long long page_stride, int n_tokens, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || !down || ld <= 0 || kv_rank <= 0 || rot_dim < 0 || rot_dims < 0 ||
      rot_dims > rot_dim || rot_dims % 2 != 0 || c_col < 0 || c_col + kv_rank + rot_dim > ld ||
      (cq && (q_rank <= 0 || q_col < 0 || q_col + q_rank > ld || !q_norm_w)) ||
      (plane && (!slots || !c_norm_w || page_size <= 0 || page_stride < (long long)page_size * (kv_rank + rot_dim))) ||
      (plane && rot_dims > 0 && (!inv_freq || !positions)))
    return ZA_ERR_ARG;
  dim3 grid(n_tokens), block(256);
  if (dtype == 0)
    hipLaunchKernelGGL((latent_prepare_kernel<float>), grid, block, 0, stream, (const float*)down,
                       ld, q_col, q_rank, c_col, kv_rank, rot_dim, q_norm_w, c_norm_w, eps,
                       positions, slots, inv_freq, rot_dims, adjacent, (float*)cq, (float*)plane,
                       page_size, page_stride);
  else if (dtype == 1)
    hipLaunchKernelGGL((latent_prepare_kernel<bf16_t>), grid, block, 0, stream,
                       (const bf16_t*)down, ld, q_col, q_rank, c_col, kv_rank, rot_dim, q_norm_w,
                       c_norm_w, eps, positions, slots, inv_freq, rot_dims, adjacent, (bf16_t*)cq,
                       (bf16_t*)plane, page_size, page_stride);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}

// --------------------------------------------------------------------- rotate_part
// dst[t][h][dst_col + i] = rotation of src[t][h][src_col + i], i < Dr (elements beyond
// rot_dims are copied).  One thread a pair.
template <typename T>
__global__ void __launch_bounds__(256)
rotate_part_kernel(const T* __restrict__ src, int src_ld, int src_col, T* __restrict__ dst,
                   int dst_ld, int dst_col, int H, int Dr, const int* __restrict__ positions,
                   const float* __restrict__ inv_freq, int rot_dims, int adjacent, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int per = Dr - rot_dims / 2;         // pairs, then the elements that pass unchanged
  const size_t th = idx / per;               // token * H + head
  const int i = (int)(idx % per);
  const T* s = src + th * src_ld + src_col;
  T* d = dst + th * dst_ld + dst_col;
  const int half = rot_dims / 2;
  if (i < half) {
    const int a = adjacent ? 2 * i : i, b = adjacent ? 2 * i + 1 : i + half;
    float sn, cs;
    sincosf((float)positions[th / H] * inv_freq[i], &sn, &cs);
    const float u = to_f32<T>(s[a]), v = to_f32<T>(s[b]);
    d[a] = from_f32<T>(u * cs - v * sn);
    d[b] = from_f32<T>(v * cs + u * sn);
  } else {
    const int e = rot_dims + (i - half);
    d[e] = s[e];
  }
}

extern "C" int za_rotate_part(const void* src, int dtype, int src_ld, int src_col, void* dst,
                              int dst_ld, int dst_col, int n_tokens, int heads, int rot_dim,
                              const int* positions, const float* inv_freq, int rot_dims,
                              int adjacent, hipStream_t stream) {
  if (n_tokens == 0 || rot_dim == 0) return 0;
  if (n_tokens < 0 || heads <= 0 || rot_dim < 0 || rot_dims < 0 || rot_dims > rot_dim ||
      rot_dims % 2 != 0 || !src || !dst || src_col < 0 || dst_col < 0 ||
      src_col + rot_dim > src_ld || dst_col + rot_dim > dst_ld ||
      (rot_dims > 0 && (!positions || !inv_freq)))
    return ZA_ERR_ARG;
  const size_t total = (size_t)n_tokens * heads * (rot_dim - rot_dims / 2);
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (dtype == 0)
    hipLaunchKernelGGL((rotate_part_kernel<float>), grid, block, 0, stream, (const float*)src,
                       src_ld, src_col, (float*)dst, dst_ld, dst_col, heads, rot_dim, positions,
                       inv_freq, rot_dims, adjacent, total);
  else if (dtype == 1)
    hipLaunchKernelGGL((rotate_part_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)src,
                       src_ld, src_col, (bf16_t*)dst, dst_ld, dst_col, heads, rot_dim, positions,
                       inv_freq, rot_dims, adjacent, total);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}

// --------------------------------------------------------------------- head_linear
// out[t][h][o_col + n] = (sum_k x[t][h][x_col + k] * W[h][n][k]) * gate(t, h, n)
//   x:   [T][H][x_ld]      W: [H][N][K]      out: [T][H][o_ld]
//   gate_mode 0: none; 1: sigmoid(gate[t][gate_col + h]); 2: sigmoid(gate[t][gate_col + h*N + n])
// Every output element is a sum over k in an order fixed by K alone.
struct HeadLinearArgs {
  const void* x;
  const void* W;
  void* out;
  const void* gate;
  int T, H, N, K;
  int x_ld, x_col, o_ld, o_col;
  int gate_ld, gate_col, gate_mode;
};

template <typename TG>
__device__ __forceinline__ float head_gate_of(const HeadLinearArgs& a, int t, int h, int n) {
  if (a.gate_mode == 0) return 1.0f;
  const TG* g = (const TG*)a.gate + (size_t)t * a.gate_ld + a.gate_col;
  const float z = to_f32<TG>(a.gate_mode == 1 ? g[h] : g[(size_t)h * a.N + n]);
  return 1.0f / (1.0f + expf(-z));
}

// bfloat16 on the matrix cores, operands straight from memory into the fragments
// (v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16), k-slots (l / 16) * 8 .. + 7 of
// either operand and receives rows (l / 16) * 4 .. + 3, column (l % 16) of the product).
// TM = 64: four waves of 16 rows x 64 columns; TM = 16 (decode batches): four waves of 16
// columns each.
template <int TM, typename TO>
__global__ void __launch_bounds__(256)
head_linear_bf16_kernel(HeadLinearArgs a) {
  constexpr int WM = TM / 16;          // waves along the rows
  constexpr int WN = 4 / WM;           // waves along the columns
  constexpr int NT = 4 / WN;           // 16-column tiles a wave
  const int h = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave % WM, wn = wave / WM;
  const int r16 = lane & 15, kq = lane >> 4;
  const int n0 = blockIdx.y * 64 + wn * NT * 16;
  const int K = a.K, N = a.N;
  const int row = blockIdx.x * TM + wm * 16 + r16;
  const bool row_ok = row < a.T;
  const bf16_t* arow = (const bf16_t*)a.x + ((size_t)(row_ok ? row : 0) * a.H + h) * a.x_ld + a.x_col;
  const bf16_t* wbase = (const bf16_t*)a.W + (size_t)h * N * K;
  const bf16_t* wrow[NT];
  bool col_ok[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = n0 + j * 16 + r16;
    col_ok[j] = n < N;
    wrow[j] = wbase + (size_t)(col_ok[j] ? n : 0) * K;
  }
  f32x4_t acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  constexpr int U = 2;
  for (int k0 = 0; k0 < K; k0 += 32 * U) {
    bf16x8_t fa[U], fw[U][NT];
#pragma unroll
    for (int s = 0; s < U; ++s) {
      const int k = k0 + s * 32 + kq * 8;
      const bool k_ok = k < K;           // K is a multiple of 8: a piece is inside or outside
      fa[s] = (row_ok && k_ok) ? *reinterpret_cast<const bf16x8_t*>(arow + k) : zero;
#pragma unroll
      for (int j = 0; j < NT; ++j)
        fw[s][j] = (col_ok[j] && k_ok) ? *reinterpret_cast<const bf16x8_t*>(wrow[j] + k) : zero;
    }
#pragma unroll
    for (int s = 0; s < U; ++s)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[s], fw[s][j], acc[j], 0, 0, 0);
  }
  TO* out = (TO*)a.out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = blockIdx.x * TM + wm * 16 + kq * 4 + i;
    if (r >= a.T) continue;
    TO* orow = out + ((size_t)r * a.H + h) * a.o_ld + a.o_col;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int n = n0 + j * 16 + r16;
      if (n < N) orow[n] = from_f32<TO>(acc[j][i] * head_gate_of<bf16_t>(a, r, h, n));
    }
  }
}

// 32-bit weights (x of either type): 64 x 64 tiles through LDS, plain FMA.
template <typename TA, typename TO>
__global__ void __launch_bounds__(256)
head_linear_f32_kernel(HeadLinearArgs a) {
  __shared__ float As[16][64 + 4];
  __shared__ float Ws[16][64 + 4];
  const int h = blockIdx.z;
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const int n0 = blockIdx.y * 64, m0 = blockIdx.x * 64;
  const int K = a.K, N = a.N;
  const float* W = (const float*)a.W + (size_t)h * N * K;
  const int lrow = tid / 4, lk = (tid % 4) * 4;
  const bool a_ok = m0 + lrow < a.T;
  const TA* arow = (const TA*)a.x + ((size_t)(a_ok ? m0 + lrow : 0) * a.H + h) * a.x_ld + a.x_col;
  const bool w_ok = n0 + lrow < N;
  const float* wrow = W + (size_t)(w_ok ? n0 + lrow : 0) * K;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      As[lk + j][lrow] = (a_ok && k < K) ? to_f32<TA>(arow[k]) : 0.f;
      Ws[lk + j][lrow] = (w_ok && k < K) ? wrow[k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
  TO* out = (TO*)a.out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = m0 + ty * 4 + i;
    if (r >= a.T) continue;
    TO* orow = out + ((size_t)r * a.H + h) * a.o_ld + a.o_col;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) orow[n] = from_f32<TO>(acc[i][j] * head_gate_of<TA>(a, r, h, n));
    }
  }
}

// dtype codes: 0 = float32, 1 = bfloat16.  The gate has x's type.
extern "C" int za_head_linear(const void* x, int x_dtype, int x_ld, int x_col, const void* W,
                              int w_dtype, void* out, int out_dtype, int o_ld, int o_col,
                              int n_tokens, int heads, int N, int K, const void* gate, int gate_ld,
                              int gate_col, int gate_mode, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || heads <= 0 || heads > 65535 || N <= 0 || K <= 0 || !x || !W || !out ||
      x_col < 0 || o_col < 0 || x_col + K > x_ld || o_col + N > o_ld || gate_mode < 0 ||
      gate_mode > 2 || (gate_mode && (!gate || gate_col < 0)) ||
      (gate_mode == 1 && gate_col + heads > gate_ld) ||
      (gate_mode == 2 && (long long)gate_col + (long long)heads * N > gate_ld))
    return ZA_ERR_ARG;
  HeadLinearArgs a{x, W, out, gate, n_tokens, heads, N, K, x_ld, x_col, o_ld, o_col,
                   gate_ld, gate_col, gate_mode};
  const unsigned ntiles = (unsigned)((N + 63) / 64);
  if (w_dtype == 1) {
    if (x_dtype != 1 || K % 8 != 0 || x_ld % 8 != 0 || x_col % 8 != 0) return ZA_ERR_UNSUPPORTED;
    const bool small = n_tokens <= 16;
    dim3 grid((unsigned)((n_tokens + (small ? 15 : 63)) / (small ? 16 : 64)), ntiles, heads);
#define ZA_HL(TMM, TO) \
  hipLaunchKernelGGL((head_linear_bf16_kernel<TMM, TO>), grid, dim3(256), 0, stream, a)
    if (out_dtype == 0) { if (small) ZA_HL(16, float); else ZA_HL(64, float); }
    else if (out_dtype == 1) { if (small) ZA_HL(16, bf16_t); else ZA_HL(64, bf16_t); }
    else return ZA_ERR_UNSUPPORTED;
#undef ZA_HL
    return za_launch_status();
  }
  if (w_dtype != 0) return ZA_ERR_UNSUPPORTED;
  dim3 grid((unsigned)((n_tokens + 63) / 64), ntiles, heads);
#define ZA_HF(TA, TO) \
  hipLaunchKernelGGL((head_linear_f32_kernel<TA, TO>), grid, dim3(256), 0, stream, a)
  if (x_dtype == 0 && out_dtype == 0) ZA_HF(float, float);
  else if (x_dtype == 1 && out_dtype == 0) ZA_HF(bf16_t, float);
  else if (x_dtype == 1 && out_dtype == 1) ZA_HF(bf16_t, bf16_t);
  else if (x_dtype == 0 && out_dtype == 1) ZA_HF(float, bf16_t);
  else return ZA_ERR_UNSUPPORTED;
#undef ZA_HF
  return za_launch_status();
}

// ---------------------------------------------------------------- latent_attention
// The general kernel: any sizes, 32-bit or bfloat16 storage, everything computed in 32-bit.
// A workgroup serves one work item (up to `count` consecutive query tokens of one request)
// and one chunk of up to LA_MAX_ROWS / count heads; a tile of KT cached rows staged in LDS
// is shared by all of them.  Rows (token, head) are dealt to the four waves; in the score
// phase a lane owns a key, in the value phase it owns latent elements.  Contexts may be cut
// into `nsplit` ranges of `keys_per_split` keys, cut at key positions that depend on nothing
// else; latent_combine merges the partial (maximum, sum, accumulator).  The sink joins the
// denominator once: at the end of a whole context here, or in the merge.
#define LA_WAVES 4
#define LA_RPW 8
#define LA_MAX_ROWS (LA_WAVES * LA_RPW)
#define LA_MAX_W 576
#define LA_MAX_R 512
#define LA_RPL (LA_MAX_R / 64)        // latent elements per lane, at most

template <typename T, int KT>
__global__ void __launch_bounds__(256)
latent_attention_kernel(const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ plane,
                        long long page_stride, const int* __restrict__ block_table, int bt_stride,
                        const int* __restrict__ positions, const int* __restrict__ wi_seq,
                        const int* __restrict__ wi_row0, const int* __restrict__ wi_count,
                        float* __restrict__ part_acc, float* __restrict__ part_ml, int H, int HC,
                        int W, int R, int page_size, float scale, int keys_per_split, int nsplit,
                        const float* __restrict__ sink) {
  extern __shared__ float smem[];
  const int ldk = W + 1;
  float* Ks = smem;                       // [KT][W + 1]
  float* Qs = Ks + KT * ldk;              // [LA_MAX_ROWS][W]
  float* Ps = Qs + LA_MAX_ROWS * W;       // [LA_WAVES][64]

  const int item = blockIdx.x, z = blockIdx.z;
  const int h0 = blockIdx.y * HC;
  const int G = min(HC, H - h0);          // heads of this chunk
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int seq = wi_seq[item];
  const int row0 = wi_row0[item];
  int count = wi_count[item];
  if (count * G > LA_MAX_ROWS) count = LA_MAX_ROWS / G;   // the host never asks for more
  const int rows = count * G;
  const int* table = block_table + (size_t)seq * bt_stride;

  const int hi = positions[row0 + count - 1];   // inclusive
  int range_lo = z * keys_per_split;
  int range_hi = range_lo + keys_per_split - 1;
  if (nsplit == 1) { range_lo = 0; range_hi = hi; }
  if (range_hi > hi) range_hi = hi;

  for (int idx = tid; idx < rows * W; idx += 256) {
    const int r = idx / W, dd = idx % W;
    const int tok = row0 + r / G, h = h0 + r % G;
    Qs[r * W + dd] = to_f32<T>(q[((size_t)tok * H + h) * W + dd]);
  }

  float m[LA_RPW], l[LA_RPW], acc[LA_RPW][LA_RPL];
#pragma unroll
  for (int i = 0; i < LA_RPW; ++i) {
    m[i] = -INFINITY;
    l[i] = 0.f;
#pragma unroll
    for (int c = 0; c < LA_RPL; ++c) acc[i][c] = 0.f;
  }

  for (int tile0 = range_lo; tile0 <= range_hi; tile0 += KT) {
    __syncthreads();  // previous tile fully consumed (and Qs written, first time)
    for (int idx = tid; idx < KT * W; idx += 256) {
      const int j = idx / W, c = idx % W;
      const int kp = tile0 + j;
      float v = 0.f;
      if (kp <= range_hi) {
        const int page = table[kp / page_size];
        if (page >= 0)
          v = to_f32<T>(plane[(size_t)page * page_stride + (size_t)(kp % page_size) * W + c]);
      }
      Ks[j * ldk + c] = v;
    }
    __syncthreads();

#pragma unroll
    for (int lr = 0; lr < LA_RPW; ++lr) {
      const int r = wave + LA_WAVES * lr;
      if (r < rows) {
        const int pos = positions[row0 + r / G];
        const int kp = tile0 + lane;
        const bool valid = lane < KT && kp <= pos && kp <= range_hi;
        float s = -INFINITY;
        if (lane < KT) {
          const float* qr = Qs + r * W;
          const float* kr = Ks + lane * ldk;
          float dot = 0.f;
          for (int dd = 0; dd < W; ++dd) dot = fmaf(qr[dd], kr[dd], dot);
          if (valid) s = dot * scale;
        }
        const float tmax = wave_max(s);
        const float m_new = fmaxf(m[lr], tmax);
        if (m_new > -INFINITY) {
          const float alpha = expf(m[lr] - m_new);
          const float p = valid ? expf(s - m_new) : 0.f;
          l[lr] = l[lr] * alpha + wave_sum(p);
          m[lr] = m_new;
          __builtin_amdgcn_wave_barrier();
          Ps[wave * 64 + lane] = p;
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int c = 0; c < LA_RPL; ++c) {
            const int dd = lane + 64 * c;
            if (64 * c < R) {
              float a = acc[lr][c] * alpha;
              if (dd < R) {
#pragma unroll 8
                for (int j = 0; j < KT; ++j) a = fmaf(Ps[wave * 64 + j], Ks[j * ldk + dd], a);
              }
              acc[lr][c] = a;
            }
          }
          __builtin_amdgcn_wave_barrier();
        }
      }
    }
  }

#pragma unroll
  for (int lr = 0; lr < LA_RPW; ++lr) {
    const int r = wave + LA_WAVES * lr;
    if (r < rows) {
      const int tok = row0 + r / G, h = h0 + r % G;
      if (nsplit == 1) {
        if (sink) l[lr] += expf(sink[h] - m[lr]);
        const float inv = l[lr] > 0.f ? 1.0f / l[lr] : 0.f;
        T* o = out + ((size_t)tok * H + h) * R;
#pragma unroll
        for (int c = 0; c < LA_RPL; ++c) {
          const int dd = lane + 64 * c;
          if (dd < R) o[dd] = from_f32<T>(acc[lr][c] * inv);
        }
      } else {
        const size_t pidx = ((size_t)tok * H + h) * nsplit + z;
        float* pa = part_acc + pidx * R;
#pragma unroll
        for (int c = 0; c < LA_RPL; ++c) {
          const int dd = lane + 64 * c;
          if (dd < R) pa[dd] = acc[lr][c];
        }
        if (lane == 0) {
          part_ml[pidx * 2] = m[lr];
          part_ml[pidx * 2 + 1] = l[lr];
        }
      }
    }
  }
}

// ------------------------------------------------------------ latent_attention_mfma
// bfloat16 on the matrix cores, rows of W and latents of R elements that are multiples of 8
// (16-byte pieces).  Per tile of 32 keys:
//   staging  every thread fetches, for 8 keys, the same 8 latent elements (eight 16-byte
//            loads), stores them as they are into Ks [32][W] and, turned round in its
//            registers, into Vt [R][32]: the second product wants, for one latent element,
//            consecutive keys side by side.  The rotated key part goes into Ks only.  The
//            loads of the next tile are issued before the products of this one.
//   S^T = K Q^T   keys are the rows of the first operand, 16 query rows the columns: a lane
//            ends up with ONE query row's scores for keys kq*4 .. +3 of each half of the
//            tile (kq = lane / 16)
//   p = 2^(s * scale * log2(e) - m) in 32-bit, the running maximum shared by the four lanes
//            of a query row; p is rounded to bfloat16 and the sum that normalises the result
//            is the sum of the rounded values
//   O^T += V^T P^T   P^T goes from the accumulator registers straight into the second
//            operand: the matrix core does not care how the 32 keys of a step are numbered
//            as long as both operands agree, so Vt holds, for lane group kq, the keys
//            kq*4 .. +3 and 16 + kq*4 .. +3 side by side at columns kq*8 .. +7
// Two kernels share this.  latent_attention_mfma_kernel: a workgroup of four waves serves
// one work item and one chunk of heads, at most 64 rows (token, head), 16 a wave.
// latent_decode_mfma_kernel: work items of at most 16 rows (single tokens times a chunk of
// 16 heads) that all four waves share: a wave takes every fourth 32-element step of the
// first product (the partial scores are added up through LDS, in a fixed order, so every
// wave holds the same scores) and every fourth 16-element tile of the result.
// Ranges of keys (`nsplit` > 1) leave (maximum on the natural scale, sum, accumulator) for
// latent_combine; the sink joins the denominator once, here or there.
// WS, RT: the most 32-element steps of a row and 16-element tiles of the latent that an
// instance holds in registers.
#define LM_KT 32
#define LM_VS (LM_KT + 8)
#define LM_NT 256
// Vt holds latent element e at row (e % 8) * P + e / 8, P = lm_vp(tiles of 16 elements): the
// threads of a wave store eight neighbouring rows each, at neighbouring e / 8, and a fragment
// reads 16 neighbouring e; with P = 2 (mod 16) and rows of 80 bytes neither meets a bank twice.
__host__ __device__ __forceinline__ int lm_vp(int rt) { return (2 * rt - 2 + 15) / 16 * 16 + 2; }
#define LM_LOG2E 1.4426950408889634f
#define LM_LN2 0.6931471805599453f

struct LmTile {
  bf16x8_t a[8];   // 8 keys x the same 8 latent elements
  bf16x8_t rot;    // 8 elements of one key's rotated part
};

struct LmCache {
  const bf16_t* plane;
  long long page_stride;
  const int* table;
  int page_size, shift;   // shift: log2(page_size), or -1
  int W, R;
};

// The page of key position `kp` (clamped into the range, so the entry exists) and the key's
// place in it: loads that depend on nothing but the tile, issued for all keys at once.
__device__ __forceinline__ int lm_page(const LmCache& c, int kp, int& off) {
  if (c.shift >= 0) {
    off = kp & (c.page_size - 1);
    return c.table[kp >> c.shift];
  }
  off = kp % c.page_size;
  return c.table[kp / c.page_size];
}

// Key `j` of the eight that lane group `g` feeds the second product side by side.
__device__ __forceinline__ int lm_key(int g, int j) { return j < 4 ? g * 4 + j : 16 + g * 4 + (j - 4); }

// No branch between the loads: a key beyond the range reads the range's last key, a page
// that is not there reads page 0, and the value is dropped afterwards.
__device__ __forceinline__ void lm_fetch(LmTile& t, const LmCache& c, int tile0, int range_hi, int tid) {
  const int nchunk = c.R / 8, rchunk = (c.W - c.R) / 8;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  if (tid < 4 * nchunk) {          // R <= 512: a block a thread at most
    const int ch = tid % nchunk, g = tid / nchunk;
    int page[8], off[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) page[j] = lm_page(c, min(tile0 + lm_key(g, j), range_hi), off[j]);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      t.a[j] = *reinterpret_cast<const bf16x8_t*>(
          c.plane + (size_t)max(page[j], 0) * c.page_stride + (size_t)off[j] * c.W + ch * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (tile0 + lm_key(g, j) > range_hi || page[j] < 0) t.a[j] = zero8;
  }
  t.rot = zero8;
  if (tid < LM_KT * rchunk) {
    const int kp = tile0 + tid / rchunk;
    int off;
    const int page = lm_page(c, min(kp, range_hi), off);
    const bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(
        c.plane + (size_t)max(page, 0) * c.page_stride + (size_t)off * c.W + c.R + (tid % rchunk) * 8);
    if (kp <= range_hi && page >= 0) t.rot = v;
  }
}

__device__ __forceinline__ void lm_store(const LmTile& t, const LmCache& c, bf16_t* Ks, bf16_t* Vt,
                                         int KS, int VP, int tile0, int range_hi, int tid) {
  const int nchunk = c.R / 8, rchunk = (c.W - c.R) / 8;
  if (tid < 4 * nchunk) {
    const int ch = tid % nchunk, g = tid / nchunk;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      *reinterpret_cast<bf16x8_t*>(Ks + lm_key(g, j) * KS + ch * 8) = t.a[j];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      bf16x8_t v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = t.a[j][r];
      *reinterpret_cast<bf16x8_t*>(Vt + (r * VP + ch) * LM_VS + g * 8) = v;
    }
  }
  if (tid < LM_KT * rchunk)
    *reinterpret_cast<bf16x8_t*>(Ks + (tid / rchunk) * KS + c.R + (tid % rchunk) * 8) = t.rot;
  // a rotated part of more than 64 elements: the rest, not fetched ahead
  for (int i = tid + LM_NT; i < LM_KT * rchunk; i += LM_NT) {
    const int key = i / rchunk, kp = tile0 + key;
    bf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (kp <= range_hi) {
      int off;
      const int page = lm_page(c, kp, off);
      if (page >= 0)
        v = *reinterpret_cast<const bf16x8_t*>(c.plane + (size_t)page * c.page_stride +
                                               (size_t)off * c.W + c.R + (i % rchunk) * 8);
    }
    *reinterpret_cast<bf16x8_t*>(Ks + key * KS + c.R + (i % rchunk) * 8) = v;
  }
}

// One query row's scores of a tile (this lane's eight keys) -> its probabilities as the
// second operand's fragment; updates the running maximum and sum; returns the factor the
// accumulator takes.
__device__ __forceinline__ float lm_softmax(const f32x4_t& s0, const f32x4_t& s1, int tile0, int kq,
                                            int pos_q, int range_hi, float scale_log2, float& m,
                                            float& l, bf16x8_t& pf) {
  float sc[8];
  float tmax = -INFINITY;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int kp = tile0 + lm_key(kq, i);
    const float v = (i < 4 ? s0[i] : s1[i - 4]) * scale_log2;
    sc[i] = (kp <= pos_q && kp <= range_hi) ? v : -INFINITY;
    tmax = fmaxf(tmax, sc[i]);
  }
  tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
  tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
  const float m_new = fmaxf(m, tmax);
  const float m_use = m_new > -INFINITY ? m_new : 0.f;
  const float alpha = m == m_new ? 1.0f : exp2f(m - m_use);
  float psum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const bf16_t pb = (bf16_t)exp2f(sc[i] - m_use);
    pf[i] = pb;
    psum += (float)pb;
  }
  l = l * alpha + psum;
  m = m_new;
  return alpha;
}

template <int WS, int RT>
__global__ void __launch_bounds__(LM_NT)
latent_attention_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                             const bf16_t* __restrict__ plane, long long page_stride,
                             const int* __restrict__ block_table, int bt_stride,
                             const int* __restrict__ positions, const int* __restrict__ wi_seq,
                             const int* __restrict__ wi_row0, const int* __restrict__ wi_count,
                             float* __restrict__ part_acc, float* __restrict__ part_ml, int H,
                             int HC, int W, int R, int page_size, int page_shift,
                             float scale_log2, int keys_per_split, int nsplit,
                             const float* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lm_lds[];
  const int ws = (W + 31) / 32, rt = (R + 15) / 16;
  const int KS = ws * 32 + 8;                       // elements from row to row of Ks
  bf16_t* Ks = reinterpret_cast<bf16_t*>(lm_lds);   // [LM_KT][KS]
  bf16_t* Vt = Ks + LM_KT * KS;                     // [8 * VP][LM_VS]
  const int VP = lm_vp(rt);

  // the last items first: within a request the later an item, the more keys it has, and
  // workgroups start in the order of their numbers, so the long ones do not start last
  const int item = gridDim.x - 1 - blockIdx.x, z = blockIdx.z;
  const int h0 = blockIdx.y * HC;
  const int G = min(HC, H - h0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kq = lane >> 4;
  const int seq = wi_seq[item];
  const int row0 = wi_row0[item];
  int count = wi_count[item];
  if (count * G > 64) count = 64 / G;               // the host never asks for more
  const int rows = count * G;
  const int hi = positions[row0 + count - 1];       // inclusive
  int range_lo = z * keys_per_split;
  int range_hi = range_lo + keys_per_split - 1;
  if (nsplit == 1) { range_lo = 0; range_hi = hi; }
  if (range_hi > hi) range_hi = hi;
  const LmCache cache = {plane, page_stride, block_table + (size_t)seq * bt_stride, page_size,
                         page_shift, W, R};

  // columns of Ks beyond W and rows of Vt beyond R stay zero: clear everything once
  {
    const int words = (LM_KT * KS + 8 * VP * LM_VS) / 2;
    uint32_t* w = reinterpret_cast<uint32_t*>(lm_lds);
    for (int i = tid; i < words; i += LM_NT) w[i] = 0u;
  }

  const int my = wave * 16 + r16;
  const bool row_ok = my < rows;
  const bool wave_on = wave * 16 < rows;
  const int tok = row0 + (row_ok ? my / G : 0);
  const int h = h0 + (row_ok ? my % G : 0);
  const int pos_q = row_ok ? positions[tok] : -1;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8_t qf[WS];
#pragma unroll
  for (int ks = 0; ks < WS; ++ks) {
    const int c = ks * 32 + kq * 8;
    qf[ks] = (row_ok && c < W)
                 ? *reinterpret_cast<const bf16x8_t*>(q + ((size_t)tok * H + h) * W + c)
                 : zero8;
  }
  float m = -INFINITY, l = 0.f;
  f32x4_t o[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) o[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  LmTile regs;
  if (range_lo <= range_hi) lm_fetch(regs, cache, range_lo, range_hi, tid);
  for (int tile0 = range_lo; tile0 <= range_hi; tile0 += LM_KT) {
    __syncthreads();      // the tile before is used up (first time: the clearing is done)
    lm_store(regs, cache, Ks, Vt, KS, VP, tile0, range_hi, tid);
    __syncthreads();
    if (tile0 + LM_KT <= range_hi) lm_fetch(regs, cache, tile0 + LM_KT, range_hi, tid);
    if (wave_on) {
      f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < WS; ++ks) {
        if (ks < ws) {
          const bf16x8_t k0 =
              *reinterpret_cast<const bf16x8_t*>(Ks + r16 * KS + ks * 32 + kq * 8);
          const bf16x8_t k1 =
              *reinterpret_cast<const bf16x8_t*>(Ks + (16 + r16) * KS + ks * 32 + kq * 8);
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qf[ks], s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qf[ks], s1, 0, 0, 0);
        }
      }
      bf16x8_t pf;
      const float alpha = lm_softmax(s0, s1, tile0, kq, pos_q, range_hi, scale_log2, m, l, pf);
      if (!__all(alpha == 1.0f)) {
#pragma unroll
        for (int t = 0; t < RT; ++t) {
          if (t < rt) { o[t][0] *= alpha; o[t][1] *= alpha; o[t][2] *= alpha; o[t][3] *= alpha; }
        }
      }
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        if (t < rt) {
          const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(
              Vt + ((r16 & 7) * VP + 2 * t + (r16 >> 3)) * LM_VS + kq * 8);
          o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[t], 0, 0, 0);
        }
      }
    }
  }

  if (!wave_on) return;
  float lt = l;
  lt += __shfl_xor(lt, 16, 64);
  lt += __shfl_xor(lt, 32, 64);
  if (!row_ok) return;
  if (nsplit == 1) {
    if (sink) lt += exp2f(sink[h] * LM_LOG2E - m);
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    bf16_t* orow = out + ((size_t)tok * H + h) * R;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int r = t * 16 + kq * 4;
      if (t < rt && r < R) {
        bf16x4_t v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (bf16_t)(o[t][i] * inv);
        *reinterpret_cast<bf16x4_t*>(orow + r) = v;
      }
    }
  } else {
    const size_t pidx = ((size_t)tok * H + h) * nsplit + z;
    float* pa = part_acc + pidx * R;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int r = t * 16 + kq * 4;
      if (t < rt && r < R) *reinterpret_cast<f32x4_t*>(pa + r) = o[t];
    }
    if (kq == 0) {
      part_ml[pidx * 2] = m * LM_LN2;
      part_ml[pidx * 2 + 1] = lt;
    }
  }
}

template <int WS, int RT>
__global__ void __launch_bounds__(LM_NT)
latent_decode_mfma_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out,
                          const bf16_t* __restrict__ plane, long long page_stride,
                          const int* __restrict__ block_table, int bt_stride,
                          const int* __restrict__ positions, const int* __restrict__ wi_seq,
                          const int* __restrict__ wi_row0, const int* __restrict__ wi_count,
                          float* __restrict__ part_acc, float* __restrict__ part_ml, int H, int HC,
                          int W, int R, int page_size, int page_shift, float scale_log2,
                          int keys_per_split, int nsplit, const float* __restrict__ sink) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lm_lds[];
  constexpr int QW = (WS + 3) / 4, OT = (RT + 3) / 4;
  const int ws = (W + 31) / 32, rt = (R + 15) / 16;
  const int KS = ws * 32 + 8;
  bf16_t* Ks = reinterpret_cast<bf16_t*>(lm_lds);   // [LM_KT][KS]
  bf16_t* Vt = Ks + LM_KT * KS;                     // [8 * VP][LM_VS]
  const int VP = lm_vp(rt);
  float* Sx = reinterpret_cast<float*>(Vt + 8 * lm_vp(rt) * LM_VS);   // [4 waves][64 lanes][8]

  const int item = blockIdx.x, z = blockIdx.z;
  const int h0 = blockIdx.y * HC;
  const int G = min(HC, H - h0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kq = lane >> 4;
  const int seq = wi_seq[item];
  const int row0 = wi_row0[item];
  int count = wi_count[item];
  if (count * G > 16) count = 16 / G;               // the host never asks for more
  const int rows = count * G;
  const int hi = positions[row0 + count - 1];       // inclusive
  int range_lo = z * keys_per_split;
  int range_hi = range_lo + keys_per_split - 1;
  if (nsplit == 1) { range_lo = 0; range_hi = hi; }
  if (range_hi > hi) range_hi = hi;
  const LmCache cache = {plane, page_stride, block_table + (size_t)seq * bt_stride, page_size,
                         page_shift, W, R};
  {
    const int words = (LM_KT * KS + 8 * VP * LM_VS) / 2;
    uint32_t* w = reinterpret_cast<uint32_t*>(lm_lds);
    for (int i = tid; i < words; i += LM_NT) w[i] = 0u;
  }

  const bool row_ok = r16 < rows;
  const int tok = row0 + (row_ok ? r16 / G : 0);
  const int h = h0 + (row_ok ? r16 % G : 0);
  const int pos_q = row_ok ? positions[tok] : -1;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8_t qf[QW];          // the steps wave, wave + 4, ... of the row
#pragma unroll
  for (int j = 0; j < QW; ++j) {
    const int c = (j * 4 + wave) * 32 + kq * 8;
    qf[j] = (row_ok && c < W)
                ? *reinterpret_cast<const bf16x8_t*>(q + ((size_t)tok * H + h) * W + c)
                : zero8;
  }
  float m = -INFINITY, l = 0.f;
  f32x4_t o[OT];            // the tiles wave, wave + 4, ... of the result
#pragma unroll
  for (int j = 0; j < OT; ++j) o[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // two tiles are on their way while one is worked on: a step of few rows has little to do
  // a tile, and what it waits for is memory
  auto tile = [&](LmTile& regs, int tile0) {
    __syncthreads();
    lm_store(regs, cache, Ks, Vt, KS, VP, tile0, range_hi, tid);
    __syncthreads();
    if (tile0 + 2 * LM_KT <= range_hi) lm_fetch(regs, cache, tile0 + 2 * LM_KT, range_hi, tid);
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < QW; ++j) {
      const int ks = j * 4 + wave;
      if (ks < ws) {
        const bf16x8_t k0 = *reinterpret_cast<const bf16x8_t*>(Ks + r16 * KS + ks * 32 + kq * 8);
        const bf16x8_t k1 =
            *reinterpret_cast<const bf16x8_t*>(Ks + (16 + r16) * KS + ks * 32 + kq * 8);
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qf[j], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qf[j], s1, 0, 0, 0);
      }
    }
    *reinterpret_cast<f32x4_t*>(Sx + (wave * 64 + lane) * 8) = s0;
    *reinterpret_cast<f32x4_t*>(Sx + (wave * 64 + lane) * 8 + 4) = s1;
    __syncthreads();
    s0 = *reinterpret_cast<const f32x4_t*>(Sx + lane * 8);
    s1 = *reinterpret_cast<const f32x4_t*>(Sx + lane * 8 + 4);
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const f32x4_t a0 = *reinterpret_cast<const f32x4_t*>(Sx + (w * 64 + lane) * 8);
      const f32x4_t a1 = *reinterpret_cast<const f32x4_t*>(Sx + (w * 64 + lane) * 8 + 4);
      s0[0] += a0[0]; s0[1] += a0[1]; s0[2] += a0[2]; s0[3] += a0[3];
      s1[0] += a1[0]; s1[1] += a1[1]; s1[2] += a1[2]; s1[3] += a1[3];
    }
    bf16x8_t pf;
    const float alpha = lm_softmax(s0, s1, tile0, kq, pos_q, range_hi, scale_log2, m, l, pf);
#pragma unroll
    for (int j = 0; j < OT; ++j) {
      const int t = j * 4 + wave;
      if (t < rt) {
        const bf16x8_t vf = *reinterpret_cast<const bf16x8_t*>(
            Vt + ((r16 & 7) * VP + 2 * t + (r16 >> 3)) * LM_VS + kq * 8);
        f32x4_t acc = o[j];
        acc[0] *= alpha; acc[1] *= alpha; acc[2] *= alpha; acc[3] *= alpha;
        o[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, acc, 0, 0, 0);
      }
    }
  };
  LmTile regs_a, regs_b;
  if (range_lo <= range_hi) lm_fetch(regs_a, cache, range_lo, range_hi, tid);
  if (range_lo + LM_KT <= range_hi) lm_fetch(regs_b, cache, range_lo + LM_KT, range_hi, tid);
  for (int tile0 = range_lo; tile0 <= range_hi; tile0 += 2 * LM_KT) {
    tile(regs_a, tile0);
    if (tile0 + LM_KT > range_hi) break;
    tile(regs_b, tile0 + LM_KT);
  }

  float lt = l;
  lt += __shfl_xor(lt, 16, 64);
  lt += __shfl_xor(lt, 32, 64);
  if (!row_ok) return;
  if (nsplit == 1) {
    if (sink) lt += exp2f(sink[h] * LM_LOG2E - m);
    const float inv = lt > 0.f ? 1.0f / lt : 0.f;
    bf16_t* orow = out + ((size_t)tok * H + h) * R;
#pragma unroll
    for (int j = 0; j < OT; ++j) {
      const int t = j * 4 + wave, r = t * 16 + kq * 4;
      if (t < rt && r < R) {
        bf16x4_t v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (bf16_t)(o[j][i] * inv);
        *reinterpret_cast<bf16x4_t*>(orow + r) = v;
      }
    }
  } else {
    const size_t pidx = ((size_t)tok * H + h) * nsplit + z;
    float* pa = part_acc + pidx * R;
#pragma unroll
    for (int j = 0; j < OT; ++j) {
      const int t = j * 4 + wave, r = t * 16 + kq * 4;
      if (t < rt && r < R) *reinterpret_cast<f32x4_t*>(pa + r) = o[j];
    }
    if (wave == 0 && kq == 0) {
      part_ml[pidx * 2] = m * LM_LN2;
      part_ml[pidx * 2 + 1] = lt;
    }
  }
}

// The partial results of a row's ranges -> the row.  `base2`: the partial maxima are whole
// numbers on the base-2 scale (what the matrix-core kernel keeps), so a partial result's
// weight 2^(m_z - m) is an exact power of two.
template <typename T>
__global__ void __launch_bounds__(64)
latent_combine_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                      T* __restrict__ out, int R, int nsplit, int base2,
                      const float* __restrict__ sink, int H) {
  const size_t row = blockIdx.x;  // token * H + head
  const int lane = threadIdx.x;
  float mx = -INFINITY;
  for (int z = 0; z < nsplit; ++z) mx = fmaxf(mx, part_ml[(row * nsplit + z) * 2]);
  float total = 0.f;
  float acc[LA_RPL];
#pragma unroll
  for (int c = 0; c < LA_RPL; ++c) acc[c] = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float mz = part_ml[(row * nsplit + z) * 2];
    const float lz = part_ml[(row * nsplit + z) * 2 + 1];
    if (!(mz > -INFINITY)) continue;
    const float w = base2 ? ldexpf(1.0f, (int)(mz - mx)) : expf(mz - mx);
    total += lz * w;
    const float* pa = part_acc + (row * nsplit + z) * R;
#pragma unroll
    for (int c = 0; c < LA_RPL; ++c) {
      const int dd = lane + 64 * c;
      if (dd < R) acc[c] = fmaf(pa[dd], w, acc[c]);
    }
  }
  if (sink && mx > -INFINITY) {
    const float sk = sink[row % H];
    total += base2 ? exp2f(sk * 1.4426950408889634f - mx) : expf(sk - mx);
  }
  const float inv = total > 0.f ? 1.0f / total : 0.f;
#pragma unroll
  for (int c = 0; c < LA_RPL; ++c) {
    const int dd = lane + 64 * c;
    if (dd < R) out[row * R + dd] = from_f32<T>(acc[c] * inv);
  }
}

template <typename T, int KT>
static int launch_latent_attention(const void* q, void* out, const void* plane,
                                   long long page_stride, const int* block_table, int bt_stride,
                                   const int* positions, const int* wi_seq, const int* wi_row0,
                                   const int* wi_count, int n_items, float* part_acc,
                                   float* part_ml, int H, int HC, int W, int R, int page_size,
                                   float scale, int keys_per_split, int nsplit, const float* sink,
                                   hipStream_t stream) {
  const size_t shmem = ((size_t)KT * (W + 1) + (size_t)LA_MAX_ROWS * W + LA_WAVES * 64) * sizeof(float);
  auto kernel = latent_attention_kernel<T, KT>;
  static size_t allowed = 0;
  if (shmem > allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (e != hipSuccess) return (int)e;
    allowed = shmem;
  }
  dim3 grid(n_items, (H + HC - 1) / HC, nsplit), block(256);
  hipLaunchKernelGGL(kernel, grid, block, shmem, stream, (const T*)q, (T*)out, (const T*)plane,
                     page_stride, block_table, bt_stride, positions, wi_seq, wi_row0, wi_count,
                     part_acc, part_ml, H, HC, W, R, page_size, scale, keys_per_split, nsplit, sink);
  return za_launch_status();
}

// The same for up to 64 ranges, a workgroup a row: the first wave turns the ranges' maxima
// and sums into weights, then every thread adds up its elements over the ranges, in the
// order of the ranges, with loads that do not wait for each other.
template <typename T>
__global__ void __launch_bounds__(256)
latent_combine_wide_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                           T* __restrict__ out, int R, int nsplit, const float* __restrict__ sink,
                           int H) {
  __shared__ float wz[64];
  __shared__ float tot;
  const size_t row = blockIdx.x;  // token * H + head
  const int tid = threadIdx.x;
  if (tid < 64) {
    float mz = -INFINITY, lz = 0.f;
    if (tid < nsplit) {
      mz = part_ml[(row * nsplit + tid) * 2];
      lz = part_ml[(row * nsplit + tid) * 2 + 1];
    }
    const float mx = wave_max(mz);
    const float w = mz > -INFINITY ? expf(mz - mx) : 0.f;
    float total = wave_sum(lz * w);
    if (sink && mx > -INFINITY) total += expf(sink[row % H] - mx);
    wz[tid] = w;
    if (tid == 0) tot = total;
  }
  __syncthreads();
  const float inv = tot > 0.f ? 1.0f / tot : 0.f;
  for (int dd = tid; dd < R; dd += 256) {
    const float* pa = part_acc + row * nsplit * R + dd;
    float acc = 0.f;
#pragma unroll 4
    for (int z = 0; z < nsplit; ++z) acc = fmaf(pa[(size_t)z * R], wz[z], acc);
    out[row * R + dd] = from_f32<T>(acc * inv);
  }
}

template <int WS, int RT, bool DECODE>
static int launch_latent_mfma(const void* q, void* out, const void* plane, long long page_stride,
                              const int* block_table, int bt_stride, const int* positions,
                              const int* wi_seq, const int* wi_row0, const int* wi_count,
                              int n_items, float* part_acc, float* part_ml, int H, int W, int R,
                              int page_size, float scale, int keys_per_split, int nsplit,
                              const float* sink, hipStream_t stream) {
  const int ws = (W + 31) / 32, rt = (R + 15) / 16;
  const size_t shmem = ((size_t)LM_KT * (ws * 32 + 8) + (size_t)8 * lm_vp(rt) * LM_VS) * sizeof(bf16_t) +
                       (DECODE ? 4 * 64 * 8 * sizeof(float) : 0);
  auto kernel = DECODE ? latent_decode_mfma_kernel<WS, RT> : latent_attention_mfma_kernel<WS, RT>;
  static size_t allowed = 0;
  if (shmem > allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (e != hipSuccess) return (int)e;
    allowed = shmem;
  }
  int shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    shift = 0;
    while ((1 << shift) < page_size) ++shift;
  }
  const int most = DECODE ? 16 : 64;
  const int HC = H < most ? H : most;
  dim3 grid(n_items, (H + HC - 1) / HC, nsplit), block(LM_NT);
  hipLaunchKernelGGL(kernel, grid, block, shmem, stream, (const bf16_t*)q, (bf16_t*)out,
                     (const bf16_t*)plane, page_stride, block_table, bt_stride, positions, wi_seq,
                     wi_row0, wi_count, part_acc, part_ml, H, HC, W, R, page_size, shift,
                     scale * LM_LOG2E, keys_per_split, nsplit, sink);
  return za_launch_status();
}

// The matrix-core form: bfloat16, `width` and `kv_rank` multiples of 8.  `waves`: 4 (work
// items of at most 64 / min(heads, 64) tokens, 16 rows a wave) or 1 (single tokens, as a
// step that only decodes has: heads in chunks of 16 whose rows the four waves share).
// Arguments otherwise as za_latent_attention.
extern "C" int za_latent_attention_mfma(const void* q, void* out, const void* plane,
                                        long long page_stride, const int* block_table,
                                        int bt_stride, const int* positions, const int* wi_seq,
                                        const int* wi_row0, const int* wi_count, int n_items,
                                        int n_tokens, float* part_acc, float* part_ml, int heads,
                                        int width, int kv_rank, int page_size, float scale,
                                        int keys_per_split, int nsplit, const float* sink,
                                        int waves, hipStream_t stream) {
  if (n_items == 0 || n_tokens == 0) return 0;
  if (n_items < 0 || heads <= 0 || width <= 0 || kv_rank <= 0 || kv_rank > width ||
      page_size <= 0 || bt_stride <= 0 || nsplit < 1 || !q || !out || !plane || !block_table ||
      !positions || !wi_seq || !wi_row0 || !wi_count ||
      page_stride < (long long)page_size * width || (waves != 1 && waves != 4))
    return ZA_ERR_ARG;
  if (width % 8 || kv_rank % 8 || width > LA_MAX_W || kv_rank > LA_MAX_R || nsplit > 65535)
    return ZA_ERR_UNSUPPORTED;
  if (nsplit > 1 && (!part_acc || !part_ml || keys_per_split <= 0 || keys_per_split % 64 != 0))
    return ZA_ERR_ARG;
  const int ws = (width + 31) / 32, rt = (kv_rank + 15) / 16;
  int rc;
#define ZA_LM_ARGS                                                                              \
  q, out, plane, page_stride, block_table, bt_stride, positions, wi_seq, wi_row0, wi_count,     \
      n_items, part_acc, part_ml, heads, width, kv_rank, page_size, scale, keys_per_split,      \
      nsplit, sink, stream
  if (ws <= 6 && rt <= 8)
    rc = waves == 4 ? launch_latent_mfma<6, 8, false>(ZA_LM_ARGS)
                    : launch_latent_mfma<6, 8, true>(ZA_LM_ARGS);
  else if (ws <= 10 && rt <= 16)
    rc = waves == 4 ? launch_latent_mfma<10, 16, false>(ZA_LM_ARGS)
                    : launch_latent_mfma<10, 16, true>(ZA_LM_ARGS);
  else
    rc = waves == 4 ? launch_latent_mfma<18, 32, false>(ZA_LM_ARGS)
                    : launch_latent_mfma<18, 32, true>(ZA_LM_ARGS);
#undef ZA_LM_ARGS
  if (rc != 0 || nsplit == 1) return rc;
  dim3 grid((unsigned)((size_t)n_tokens * heads));
  if (nsplit <= 64)
    hipLaunchKernelGGL((latent_combine_wide_kernel<bf16_t>), grid, dim3(256), 0, stream, part_acc,
                       part_ml, (bf16_t*)out, kv_rank, nsplit, sink, heads);
  else
    hipLaunchKernelGGL((latent_combine_kernel<bf16_t>), grid, dim3(64), 0, stream, part_acc,
                       part_ml, (bf16_t*)out, kv_rank, nsplit, 0, sink, heads);
  return za_launch_status();
}

// q: [T][H][W] folded queries; out: [T][H][R]; plane: the cache, a page's rows one after
// the other, `page_stride` elements from page to page.  Work items: (request, first row,
// rows), each with at most LA_MAX_ROWS / min(H, LA_MAX_ROWS) rows.
extern "C" int za_latent_attention(const void* q, void* out, const void* plane,
                                   long long page_stride, const int* block_table, int bt_stride,
                                   const int* positions, const int* wi_seq, const int* wi_row0,
                                   const int* wi_count, int n_items, int n_tokens, float* part_acc,
                                   float* part_ml, int dtype, int heads, int width, int kv_rank,
                                   int page_size, float scale, int keys_per_split, int nsplit,
                                   const float* sink, hipStream_t stream) {
  if (n_items == 0 || n_tokens == 0) return 0;
  if (n_items < 0 || heads <= 0 || width <= 0 || kv_rank <= 0 || kv_rank > width ||
      page_size <= 0 || bt_stride <= 0 || nsplit < 1 || !q || !out || !plane || !block_table ||
      !positions || !wi_seq || !wi_row0 || !wi_count ||
      page_stride < (long long)page_size * width)
    return ZA_ERR_ARG;
  if (width > LA_MAX_W || kv_rank > LA_MAX_R || nsplit > 65535) return ZA_ERR_UNSUPPORTED;
  if (nsplit > 1 && (!part_acc || !part_ml || keys_per_split <= 0 || keys_per_split % 64 != 0))
    return ZA_ERR_ARG;
  const int HC = heads < LA_MAX_ROWS ? heads : LA_MAX_ROWS;
  int rc;
#define ZA_LA_ARGS                                                                             \
  q, out, plane, page_stride, block_table, bt_stride, positions, wi_seq, wi_row0, wi_count,    \
      n_items, part_acc, part_ml, heads, HC, width, kv_rank, page_size, scale, keys_per_split, \
      nsplit, sink, stream
  const bool small = width <= 256;
  if (dtype == 0)
    rc = small ? launch_latent_attention<float, 64>(ZA_LA_ARGS)
               : launch_latent_attention<float, 32>(ZA_LA_ARGS);
  else if (dtype == 1)
    rc = small ? launch_latent_attention<bf16_t, 64>(ZA_LA_ARGS)
               : launch_latent_attention<bf16_t, 32>(ZA_LA_ARGS);
  else
    return ZA_ERR_UNSUPPORTED;
#undef ZA_LA_ARGS
  if (rc != 0 || nsplit == 1) return rc;
  dim3 grid((unsigned)((size_t)n_tokens * heads)), block(64);
  if (dtype == 0)
    hipLaunchKernelGGL((latent_combine_kernel<float>), grid, block, 0, stream, part_acc, part_ml,
                       (float*)out, kv_rank, nsplit, 0, sink, heads);
  else
    hipLaunchKernelGGL((latent_combine_kernel<bf16_t>), grid, block, 0, stream, part_acc, part_ml,
                       (bf16_t*)out, kv_rank, nsplit, 0, sink, heads);
  return za_launch_status();
}
