// A feed-forward of many small experts of which each token uses a few: the lists of
// who goes where, and products of every expert's rows with that expert's weights in one
// launch ("grouped" products).
//
// A step has A = T * top assignments; assignment a = t * top + j is token t's j-th expert.
//
// 1. expert_lists: one workgroup an expert walks the assignments in order and writes the
//    ones that name it, ascending, into lists[e][0 .. counts[e]).  No atomics, nothing to
//    clear beforehand, and the lists do not depend on the order in which anything ran.
//    Where an expert comes from is the caller's business: here a table indexed by the
//    token id, [vocab][top] (a router's top-k output [T][top] takes the same kernel with
//    the row index in place of the token id).
//
// 2. grouped_gemm: for every expert e and every tile of TM of its assignments,
//        out[dst(a)] = f(src[a / src_div] @ W[e]^T) * out_scale
//    src_div = top reads the tokens' rows, src_div = 1 rows that are already one an
//    assignment.  dst(a) = a, or, `stacked`, (a % top) * T + a / top: a stack [top][T][N]
//    of 32-bit partial results, which the norm that follows adds up in its order (so the
//    weighted sum over a token's experts is taken in 32-bit and costs no kernel).
//    f: nothing, or the square of relu.
//    How many tiles there are is known on the device only; the grid is the upper bound
//    ceil(A / TM) + E and a workgroup beyond the last tile leaves at once.
//    Every output element is a sum over k in an order fixed by K alone: a token's result
//    does not depend on which other tokens share its expert or its tile.
//      bfloat16: matrix cores (v_mfma_f32_16x16x32_bf16), operands straight from memory
//      into the fragments; TM = 64 (four waves, 16 rows x 64 columns each) for steps with
//      prompt portions, TM = 16 (four waves, 16 columns each) for decode batches, where an
//      expert has a token or two and the weights are all that moves; for steps of many
//      tokens an expert (128 and more on average) tiles of 128 x 128 through LDS, a step of
//      64 of K at a time with the next step's pieces on their way into registers, four
//      waves of 64 x 64 each: every element of either operand is then read from memory
//      once a tile and used 128 times.
//      32-bit: LDS-tiled FMA, 64 x 64 tiles (no matrix-core rounding mode).
#include "common.h"

#define EX_MAX_EXPERTS 1024

// lists: int [E][A]; counts: int [E].  `ids` names the table's row for each token (null:
// the token's own index); an id outside [0, rows) names no expert.
__global__ void __launch_bounds__(256)
expert_lists_kernel(const int* __restrict__ ids, const int* __restrict__ table, int rows, int T,
                    int top, int* __restrict__ lists, int* __restrict__ counts) {
  __shared__ int wave_total[4];
  const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int A = T * top;
  int* mine = lists + (size_t)e * A;
  int running = 0;
  for (int base = 0; base < A; base += 256) {
    const int a = base + tid;
    bool hit = false;
    if (a < A) {
      const int t = a / top, id = ids ? ids[t] : t;
      hit = id >= 0 && id < rows && table[(size_t)id * top + a % top] == e;
    }
    const unsigned long long mask = __ballot(hit);
    const int before = __popcll(mask & ((1ull << lane) - 1ull));
    __syncthreads();      // the totals of the chunk before have been read
    if (lane == 0) wave_total[wave] = __popcll(mask);
    __syncthreads();
    int offset = running;
    for (int w = 0; w < wave; ++w) offset += wave_total[w];
    if (hit) mine[offset + before] = a;
    running += wave_total[0] + wave_total[1] + wave_total[2] + wave_total[3];
  }
  if (tid == 0) counts[e] = running;
}

extern "C" int za_expert_lists(const int* ids, const int* table, int rows, int n_tokens, int top,
                               int experts, int* lists, int* counts, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || top <= 0 || experts <= 0 || rows <= 0 || !table || !lists || !counts)
    return ZA_ERR_ARG;
  if (experts > EX_MAX_EXPERTS) return ZA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(expert_lists_kernel, dim3(experts), dim3(256), 0, stream, ids, table, rows,
                     n_tokens, top, lists, counts);
  return za_launch_status();
}

struct GroupedArgs {
  const void* src;       // [rows][K]
  const void* W;         // [E][N][K]
  const int* lists;      // [E][A]
  const int* counts;     // [E]
  void* out;
  int A, T, top, E, N, K;
  int src_div, stacked, act;
  float out_scale;
};

// The expert and the tile within it that workgroup `b` serves; false when there is none.
template <int TM>
__device__ __forceinline__ bool find_tile(const int* __restrict__ counts, int E, int b, int* e_out,
                                          int* tile_out, int* count_out) {
  int first = 0;
  for (int e = 0; e < E; ++e) {
    const int c = counts[e], tiles = (c + TM - 1) / TM;
    if (b < first + tiles) {
      *e_out = e;
      *tile_out = b - first;
      *count_out = c;
      return true;
    }
    first += tiles;
  }
  return false;
}

__device__ __forceinline__ float expert_act(float v, int act) {
  if (act == 1) {
    const float r = fmaxf(v, 0.f);
    return r * r;
  }
  return v;
}

__device__ __forceinline__ size_t dst_row(const GroupedArgs& g, int a) {
  return g.stacked ? (size_t)(a % g.top) * g.T + a / g.top : (size_t)a;
}

// Operand layout of v_mfma_f32_16x16x32_bf16: lane l supplies row (l % 16), k-slots
// (l / 16) * 8 .. + 7 of either operand and receives rows (l / 16) * 4 .. + 3, column
// (l % 16) of the product.
template <int TM, typename TO>
__global__ void __launch_bounds__(256)
grouped_gemm_bf16_kernel(GroupedArgs g) {
  constexpr int WM = TM / 16;          // waves along the rows
  constexpr int WN = 4 / WM;           // waves along the columns
  constexpr int NT = 4 / WN;           // 16-column tiles a wave
  int e, tile, count;
  if (!find_tile<TM>(g.counts, g.E, blockIdx.x, &e, &tile, &count)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave % WM, wn = wave / WM;
  const int r16 = lane & 15, kq = lane >> 4;
  const int n0 = blockIdx.y * 64 + wn * NT * 16;
  const int* mine = g.lists + (size_t)e * g.A;
  const int K = g.K, N = g.N;

  const int row = tile * TM + wm * 16 + r16;
  const bool row_ok = row < count;
  const bf16_t* arow = (const bf16_t*)g.src + (size_t)(row_ok ? mine[row] / g.src_div : 0) * K;
  const bf16_t* wbase = (const bf16_t*)g.W + (size_t)e * N * K;
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

  // steps of 32 at a time (two, or four where a wave has one column tile: a decode batch,
  // which only streams weights): their loads are all requested before the first product
  constexpr int U = NT == 1 ? 4 : 2;
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

  TO* out = (TO*)g.out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * TM + wm * 16 + kq * 4 + i;
    if (r >= count) continue;
    const size_t d = dst_row(g, mine[r]);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int n = n0 + j * 16 + r16;
      if (n < N) out[d * N + n] = from_f32<TO>(expert_act(acc[j][i], g.act) * g.out_scale);
    }
  }
}

// Tiles of 128 assignments x 128 outputs through LDS, for experts with many rows.
#define GG_BM 128
#define GG_BN 128
#define GG_BK 64
#define GG_LD (GG_BK + 8)   // padded row, in elements: spreads rows over LDS banks

#ifndef GG_MIN_WAVES
#define GG_MIN_WAVES 2    // waves a SIMD the register budget is cut for
#endif

template <typename TO>
__global__ void __launch_bounds__(256, GG_MIN_WAVES)
grouped_gemm_bf16_tiled_kernel(GroupedArgs g) {
  __shared__ __attribute__((aligned(16))) bf16_t As[GG_BM * GG_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[GG_BN * GG_LD];
  int e, tile, count;
  if (!find_tile<GG_BM>(g.counts, g.E, blockIdx.x, &e, &tile, &count)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int n0 = blockIdx.y * GG_BN;
  const int* mine = g.lists + (size_t)e * g.A;
  const int K = g.K, N = g.N;
  const bf16_t* wbase = (const bf16_t*)g.W + (size_t)e * N * K;

  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // a thread moves 4 + 4 pieces of 8 elements a step: rows lrow + 32 i, elements lcol .. + 7
  const int lrow = tid >> 3, lcol = (tid & 7) * 8;
  const bf16_t* arow[4];
  const bf16_t* wrow[4];
  bool a_ok[4], w_ok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * GG_BM + lrow + 32 * i, n = n0 + lrow + 32 * i;
    a_ok[i] = r < count;
    w_ok[i] = n < N;
    arow[i] = (const bf16_t*)g.src + (size_t)(a_ok[i] ? mine[r] / g.src_div : 0) * K;
    wrow[i] = wbase + (size_t)(w_ok[i] ? n : 0) * K;
  }
  bf16x8_t ra[4], rw[4];
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  auto fetch = [&](int k0) {
    const int k = k0 + lcol;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[i] = (a_ok[i] && k < K) ? *reinterpret_cast<const bf16x8_t*>(arow[i] + k) : zero8;
      rw[i] = (w_ok[i] && k < K) ? *reinterpret_cast<const bf16x8_t*>(wrow[i] + k) : zero8;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<bf16x8_t*>(As + (lrow + 32 * i) * GG_LD + lcol) = ra[i];
      *reinterpret_cast<bf16x8_t*>(Ws + (lrow + 32 * i) * GG_LD + lcol) = rw[i];
    }
  };
  fetch(0);
  stash();
  __syncthreads();
  const int r16 = lane & 15, kq = (lane >> 4) * 8;
  for (int k0 = 0; k0 < K; k0 += GG_BK) {
    const bool more = k0 + GG_BK < K;
    if (more) fetch(k0 + GG_BK);
#pragma unroll
    for (int ks = 0; ks < GG_BK; ks += 32) {
      bf16x8_t fa[4], fw[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        fa[i] = *reinterpret_cast<const bf16x8_t*>(As + (wm * 64 + i * 16 + r16) * GG_LD + ks + kq);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        fw[j] = *reinterpret_cast<const bf16x8_t*>(Ws + (wn * 64 + j * 16 + r16) * GG_LD + ks + kq);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
    if (more) {
      stash();
      __syncthreads();
    }
  }
  TO* out = (TO*)g.out;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = tile * GG_BM + wm * 64 + i * 16 + (lane >> 4) * 4 + r;
      if (row >= count) continue;
      const size_t d = dst_row(g, mine[row]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + wn * 64 + j * 16 + r16;
        if (n < N) out[d * N + n] = from_f32<TO>(expert_act(acc[i][j][r], g.act) * g.out_scale);
      }
    }
}

// 32-bit weights (src of either type): 64 x 64 tiles through LDS, plain FMA.
template <typename TA, typename TO>
__global__ void __launch_bounds__(256)
grouped_gemm_f32_kernel(GroupedArgs g) {
  __shared__ float As[16][64 + 4];
  __shared__ float Ws[16][64 + 4];
  int e, tile, count;
  if (!find_tile<64>(g.counts, g.E, blockIdx.x, &e, &tile, &count)) return;
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const int n0 = blockIdx.y * 64;
  const int* mine = g.lists + (size_t)e * g.A;
  const int K = g.K, N = g.N;
  const float* W = (const float*)g.W + (size_t)e * N * K;
  const int lrow = tid / 4, lk = (tid % 4) * 4;
  const int arow_idx = tile * 64 + lrow;
  const bool a_ok = arow_idx < count;
  const TA* arow = (const TA*)g.src + (size_t)(a_ok ? mine[arow_idx] / g.src_div : 0) * K;
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
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
  TO* out = (TO*)g.out;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tile * 64 + ty * 4 + i;
    if (r >= count) continue;
    const size_t d = dst_row(g, mine[r]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[d * N + n] = from_f32<TO>(expert_act(acc[i][j], g.act) * g.out_scale);
    }
  }
}

// dtype codes: 0 = float32, 1 = bfloat16.  `src` has `src_rows` rows of K elements; the
// lists name assignments below n_tokens * top, so src_rows >= n_tokens (src_div == top) or
// >= n_tokens * top (src_div == 1).
extern "C" int za_grouped_gemm(const void* src, int src_dtype, long long src_rows, const void* W,
                               int w_dtype, const int* lists, const int* counts, void* out,
                               int out_dtype, int n_tokens, int top, int experts, int N, int K,
                               int src_div, int stacked, int act, float out_scale,
                               hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || top <= 0 || experts <= 0 || N <= 0 || K <= 0 || !src || !W || !lists ||
      !counts || !out || (src_div != 1 && src_div != top) || act < 0 || act > 1)
    return ZA_ERR_ARG;
  const long long A = (long long)n_tokens * top;
  if (src_rows < (src_div == 1 ? A : (long long)n_tokens) || A > 0x7fffffff) return ZA_ERR_ARG;
  if (experts > EX_MAX_EXPERTS) return ZA_ERR_UNSUPPORTED;
  if (stacked && out_dtype != 0) return ZA_ERR_UNSUPPORTED;
  GroupedArgs g{src, W, lists, counts, out, (int)A, n_tokens, top, experts, N, K,
                src_div, stacked, act, out_scale};
  const unsigned ntiles = (unsigned)((N + 63) / 64);
  if (w_dtype == 1) {
    if (src_dtype != 1 || K % 8 != 0) return ZA_ERR_UNSUPPORTED;
    if (A >= 128LL * experts) {
      // many rows an expert: tiles of 128 x 128 through LDS
      dim3 grid((unsigned)((A + GG_BM - 1) / GG_BM + experts), (unsigned)((N + GG_BN - 1) / GG_BN));
      if (out_dtype == 0)
        hipLaunchKernelGGL((grouped_gemm_bf16_tiled_kernel<float>), grid, dim3(256), 0, stream, g);
      else if (out_dtype == 1)
        hipLaunchKernelGGL((grouped_gemm_bf16_tiled_kernel<bf16_t>), grid, dim3(256), 0, stream, g);
      else
        return ZA_ERR_UNSUPPORTED;
      return za_launch_status();
    }
    // a decode batch (an expert has a token or two): tiles of 16 rows
    const bool small = A <= 4LL * experts || A <= 64;
    const int TM = small ? 16 : 64;
    dim3 grid((unsigned)((A + TM - 1) / TM + experts), ntiles), block(256);
#define ZA_GG(TMM, TO) \
  hipLaunchKernelGGL((grouped_gemm_bf16_kernel<TMM, TO>), grid, block, 0, stream, g)
    if (out_dtype == 0) { if (small) ZA_GG(16, float); else ZA_GG(64, float); }
    else if (out_dtype == 1) { if (small) ZA_GG(16, bf16_t); else ZA_GG(64, bf16_t); }
    else return ZA_ERR_UNSUPPORTED;
#undef ZA_GG
    return za_launch_status();
  }
  if (w_dtype != 0) return ZA_ERR_UNSUPPORTED;
  dim3 grid((unsigned)((A + 63) / 64 + experts), ntiles), block(256);
#define ZA_GF(TA, TO) \
  hipLaunchKernelGGL((grouped_gemm_f32_kernel<TA, TO>), grid, block, 0, stream, g)
  if (src_dtype == 0 && out_dtype == 0) ZA_GF(float, float);
  else if (src_dtype == 1 && out_dtype == 0) ZA_GF(bf16_t, float);
  else if (src_dtype == 1 && out_dtype == 1) ZA_GF(bf16_t, bf16_t);
  else if (src_dtype == 0 && out_dtype == 1) ZA_GF(float, bf16_t);
  else return ZA_ERR_UNSUPPORTED;
#undef ZA_GF
  return za_launch_status();
}

// ------------------------------------------------------------------------ a router
// Which `top` of `n` router outputs every token uses, and with which weight.  One wave a
// token, everything in 32-bit:
//   s = softmax(z) over all n outputs (mode 0) or sigmoid(z) (mode 1)
//   c = s + correction          the choice score (correction may be absent)
//   the outputs form `groups` equal groups of neighbours; a group's score is its largest c,
//   and only outputs of the `keep` best groups can be chosen (the others count as minus
//   infinity); groups == 0: no such limit
//   chosen = the `top` outputs with the largest c, in descending order (of equal scores the
//   lower index first); weight = s[chosen] * scale, or, `renorm`, divided by the sum of
//   the chosen s first
// What an output beyond the experts that have weights means (an expert that hands its input
// on, say) is the business of whoever reads `chosen`.
#define RT_MAX 1024

__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int o = ZA_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, ZA_WAVE);
    const int oi = __shfl_xor(i, o, ZA_WAVE);
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
  }
}

__global__ void __launch_bounds__(64)
route_topk_kernel(const float* __restrict__ z, int ld, const float* __restrict__ correction, int n,
                  int groups, int keep, int top, float scale, int mode, int renorm,
                  int* __restrict__ chosen, float* __restrict__ weight) {
  __shared__ float ss[RT_MAX], cs[RT_MAX], gs[RT_MAX];
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* zr = z + (size_t)t * ld;
  if (mode == 0) {
    float mx = -INFINITY;
    for (int e = lane; e < n; e += 64) mx = fmaxf(mx, zr[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < n; e += 64) {
      const float p = expf(zr[e] - mx);
      ss[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    for (int e = lane; e < n; e += 64) ss[e] *= inv;
  } else {
    for (int e = lane; e < n; e += 64) ss[e] = 1.0f / (1.0f + expf(-zr[e]));
  }
  for (int e = lane; e < n; e += 64) cs[e] = ss[e] + (correction ? correction[e] : 0.f);
  __builtin_amdgcn_wave_barrier();
  __syncthreads();
  if (groups > 1 && keep < groups) {
    const int per = n / groups;
    for (int g = lane; g < groups; g += 64) {
      float best = -INFINITY;
      for (int k = 0; k < per; ++k) best = fmaxf(best, cs[g * per + k]);
      gs[g] = best;
    }
    __syncthreads();
    // the `keep` best groups get the mark +inf; afterwards every other group is closed
    for (int r = 0; r < keep; ++r) {
      float v = -INFINITY;
      int at = 0x7fffffff;
      for (int g = lane; g < groups; g += 64) {
        const float x = gs[g];
        if (x != INFINITY && (x > v || (x == v && g < at))) { v = x; at = g; }
      }
      wave_argmax(v, at);
      __syncthreads();
      if (lane == 0 && at < groups) gs[at] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < n; e += 64)
      if (gs[e / per] != INFINITY) cs[e] = -INFINITY;
    __syncthreads();
  }
  float total = 0.f;
  for (int j = 0; j < top; ++j) {
    float v = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < n; e += 64) {
      const float x = cs[e];
      // (a taken output holds NaN, which compares false)
      if (x > v || (x == v && e < at)) { v = x; at = e; }
    }
    wave_argmax(v, at);
    __syncthreads();
    if (at >= n) at = 0;      // nothing left to choose from: cannot happen with top <= open outputs
    const float s = ss[at];
    total += s;
    if (lane == 0) {
      chosen[(size_t)t * top + j] = at;
      weight[(size_t)t * top + j] = s;
      cs[at] = __builtin_nanf("");
    }
    __syncthreads();
  }
  const float f = renorm ? scale / total : scale;
  for (int j = lane; j < top; j += 64) weight[(size_t)t * top + j] *= f;
}

extern "C" int za_route_topk(const float* z, int ld, const float* correction, int n_tokens, int n,
                             int groups, int keep, int top, float scale, int mode, int renorm,
                             int* chosen, float* weight, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || n <= 0 || ld < n || top <= 0 || top > n || !z || !chosen || !weight ||
      groups < 0 || (groups > 0 && (n % groups != 0 || keep <= 0 || keep > groups)) ||
      mode < 0 || mode > 1)
    return ZA_ERR_ARG;
  if (groups > 0 && (long long)keep * (n / groups) < top) return ZA_ERR_ARG;
  if (n > RT_MAX) return ZA_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(route_topk_kernel, dim3(n_tokens), dim3(64), 0, stream, z, ld, correction, n,
                     groups, keep, top, scale, mode, renorm, chosen, weight);
  return za_launch_status();
}

// What a token's chosen experts and the shared expert give, as one 32-bit row:
//   y[t] = sum_j weight[t][j] * (chosen[t][j] < n_real ? expert_out[t * top + j] : x[t])
//          + gate(t) * shared[t]
// An output beyond the n_real experts that have weights hands the token's input x[t] on.
// gate(t) = sigmoid(gate_logits[t * gate_ld]) when gate_logits is given, else 1; `shared`
// may be absent.  The sum is taken in the order j = 0 .. top - 1, then the shared expert.
template <typename TE, typename TX>
__global__ void __launch_bounds__(256)
experts_combine_kernel(const TE* __restrict__ expert_out, const int* __restrict__ chosen,
                       const float* __restrict__ weight, const TX* __restrict__ x,
                       const TE* __restrict__ shared, const float* __restrict__ gate_logits,
                       int gate_ld, float* __restrict__ y, int top, int n_real, int width) {
  const size_t t = blockIdx.x;
  float g = 1.0f;
  if (shared && gate_logits) g = 1.0f / (1.0f + expf(-gate_logits[t * gate_ld]));
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = chosen[t * top + j];
      const float w = weight[t * top + j];
      const float v = e < n_real ? to_f32<TE>(expert_out[(t * top + j) * width + i])
                                 : to_f32<TX>(x[t * width + i]);
      acc = fmaf(w, v, acc);
    }
    if (shared) acc = fmaf(g, to_f32<TE>(shared[t * width + i]), acc);
    y[t * width + i] = acc;
  }
}

// dtype codes: 0 = float32, 1 = bfloat16; `out_dtype` is that of expert_out and shared.
extern "C" int za_experts_combine(const void* expert_out, int out_dtype, const int* chosen,
                                  const float* weight, const void* x, int x_dtype,
                                  const void* shared, const float* gate_logits, int gate_ld,
                                  float* y, int n_tokens, int top, int n_real, int width,
                                  hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || top <= 0 || width <= 0 || n_real < 0 || !chosen || !weight || !x || !y ||
      (n_real > 0 && !expert_out))
    return ZA_ERR_ARG;
  dim3 grid(n_tokens), block(width <= 256 ? 64 : 256);
#define ZA_EC(TE, TX)                                                                          \
  hipLaunchKernelGGL((experts_combine_kernel<TE, TX>), grid, block, 0, stream,                 \
                     (const TE*)expert_out, chosen, weight, (const TX*)x, (const TE*)shared,   \
                     gate_logits, gate_ld, y, top, n_real, width)
  if (out_dtype == 0 && x_dtype == 0) ZA_EC(float, float);
  else if (out_dtype == 0 && x_dtype == 1) ZA_EC(float, bf16_t);
  else if (out_dtype == 1 && x_dtype == 1) ZA_EC(bf16_t, bf16_t);
  else if (out_dtype == 1 && x_dtype == 0) ZA_EC(bf16_t, float);
  else return ZA_ERR_UNSUPPORTED;
#undef ZA_EC
  return za_launch_status();
}
