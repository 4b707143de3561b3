// Mixers that carry a matrix state from token to token, for any mix of prompt
// portions and single decoded tokens in one launch.  Everything that enters a
// recurrence is 32-bit: the state, decays, step sizes, gates and unit norms.
//
// 1. causal_conv_silu: a depth-wise causal convolution over a request's own inputs
//    followed by silu (or, through za_causal_conv, by nothing),
//      y[t, c] = silu(bias[c] + sum_j taps[c, j] * x[t - (L - 1 - j), c]),
//    the L - 1 inputs before a portion coming from the request's state slot, which
//    afterwards holds the portion's last L - 1 inputs.
//
// 2. matrix_recurrence, per (request, head), with a state S of `dk` rows (key
//    channels) and `dv` columns, in two forms:
//      SSD (state-space duality):   S <- a S + dt * b x^T;          y = S^T c + D x
//          a = exp(-exp(A_log) * dt), dt = softplus(raw + dt_bias)      (one per head)
//      gated delta rule:            S <- diag(g) S;  u = beta (v - S^T k);
//                                   S <- S + k u^T;  o = S^T q
//          g = exp(-exp(A_log) * softplus(raw + dt_bias))   (one per head and key channel)
//          q, k made unit vectors (x / sqrt(sum x^2 + 1e-6)), q times dk^(-1/2),
//          beta = sigmoid(raw)
//      fixed decay (retention):      S <- a_h S + k v^T;             o = S^T q
//          a_h a constant of the head; the SSD walk with dt = 1 and no D, q and k rotated
//          and k scaled beforehand by retention_prepare
//    A column of S never meets another column: P neighbouring lanes that split its rows
//    keep one column in registers across all tokens of the portion, read it from the
//    slot at the start and store it at the end.  The slot holds S turned round,
//    [head][column][row], so that a lane's rows are consecutive floats.  What a token
//    brings that does not depend on the state (unit vectors, decays, gates) is computed
//    beforehand, for all tokens at once; a workgroup is one wave that walks the tokens in
//    order with the next tokens' vectors already on their way.
//
// 3. gated_group_norm: y * act(gate) and an RMS norm over equal groups of columns, the
//    gate before or after the norm:
//      gate first:  v = y * act(gate);  out = v / rms(v) * w
//      gate last:   out = y / rms(y) * w * act(gate)
#include <math.h>

#include "common.h"
#include "rope_math.h"

#define RC_MAX_TAPS 8

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
// log(1 + exp(x)) without overflow; no clamp
__device__ __forceinline__ float softplus_f(float x) {
  return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
}

// ------------------------------------------------------------------ convolution
// grid.x: blocks of 256 channels; grid.y: first the blocks of `tokens_per_block`
// tokens (bodies: tokens whose L - 1 predecessors lie in the same portion), then one
// block per request (heads: the first L - 1 tokens of its portion and the state).
// `act`: 1 silu, 0 none.  `TO`: what is stored (the state keeps 32-bit inputs either way).
template <typename T, typename TO>
__global__ void __launch_bounds__(256)
causal_conv_silu_kernel(const T* __restrict__ x, int x_stride, int col0,
                        const float* __restrict__ taps, const float* __restrict__ bias,
                        float* __restrict__ state, long long slot_stride,
                        const int* __restrict__ token_seq, const int* __restrict__ seq_start,
                        const int* __restrict__ slot_id, TO* __restrict__ out, int n_tokens,
                        int C, int L, int body_blocks, int tokens_per_block, int act) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  float w[RC_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < RC_MAX_TAPS; ++j) w[j] = j < L ? taps[(size_t)c * L + j] : 0.f;
  const float b = bias ? bias[c] : 0.f;
  if ((int)blockIdx.y < body_blocks) {
    const int t0 = blockIdx.y * tokens_per_block;
    // the L - 1 inputs before the token stay in registers from one token to the next
    float before[RC_MAX_TAPS];
    bool have = false;
    for (int t = t0; t < t0 + tokens_per_block && t < n_tokens; ++t) {
      const int rel = t - seq_start[token_seq[t]];
      if (rel < L - 1) {
        have = false;
        continue;
      }
      if (!have) {
#pragma unroll
        for (int j = 0; j < RC_MAX_TAPS - 1; ++j)
          before[j] = j < L - 1 ? to_f32<T>(x[(size_t)(t - (L - 1 - j)) * x_stride + col0 + c]) : 0.f;
        have = true;
      }
      const float xi = to_f32<T>(x[(size_t)t * x_stride + col0 + c]);
      float acc = b;
#pragma unroll
      for (int j = 0; j < RC_MAX_TAPS - 1; ++j)
        if (j < L - 1) acc = fmaf(w[j], before[j], acc);
      acc = fmaf(w[L - 1], xi, acc);
      out[(size_t)t * C + c] = from_f32<TO>(act ? silu_f(acc) : acc);
#pragma unroll
      for (int j = 0; j < RC_MAX_TAPS - 1; ++j)
        if (j < L - 2) before[j] = before[j + 1];
      if (L >= 2) before[L - 2] = xi;
    }
    return;
  }
  const int s = blockIdx.y - body_blocks;
  const int start = seq_start[s], n = seq_start[s + 1] - start;
  float* st = state + (size_t)slot_id[s] * slot_stride + (size_t)c * (L - 1);
  float hist[RC_MAX_TAPS];      // the L - 1 inputs before the next token, oldest first
#pragma unroll
  for (int j = 0; j < RC_MAX_TAPS; ++j) hist[j] = j < L - 1 ? st[j] : 0.f;
  const int first = n < L - 1 ? n : L - 1;
  for (int i = 0; i < first; ++i) {
    const float xi = to_f32<T>(x[(size_t)(start + i) * x_stride + col0 + c]);
    float acc = b;
#pragma unroll
    for (int j = 0; j < RC_MAX_TAPS - 1; ++j)
      if (j < L - 1) acc = fmaf(w[j], hist[j], acc);
    acc = fmaf(w[L - 1], xi, acc);
    out[(size_t)(start + i) * C + c] = from_f32<TO>(act ? silu_f(acc) : acc);
#pragma unroll
    for (int j = 0; j < RC_MAX_TAPS - 1; ++j)
      if (j < L - 2) hist[j] = hist[j + 1];
    if (L >= 2) hist[L - 2] = xi;
  }
  if (n > L - 1) {
#pragma unroll
    for (int j = 0; j < RC_MAX_TAPS; ++j)
      if (j < L - 1)
        hist[j] = to_f32<T>(x[(size_t)(start + n - (L - 1) + j) * x_stride + col0 + c]);
  }
#pragma unroll
  for (int j = 0; j < RC_MAX_TAPS; ++j)
    if (j < L - 1) st[j] = hist[j];
}

// `act`: 1 silu, 0 none; `out_dtype`: 0 the result as 32-bit floats, 1 as bfloat16.
extern "C" int za_causal_conv(const void* x, int dtype, int x_stride, int col0, const float* taps,
                              const float* bias, float* state, long long slot_stride,
                              const int* token_seq, const int* seq_start, const int* slot_id,
                              void* out, int out_dtype, int act, int n_tokens, int n_seqs, int C,
                              int L, hipStream_t stream) {
  if (n_tokens == 0 || n_seqs == 0) return 0;
  if (n_tokens < 0 || n_seqs < 0 || C <= 0 || !x || !taps || !state || !token_seq || !seq_start ||
      !slot_id || !out || col0 < 0 || col0 + C > x_stride || slot_stride < (long long)C * (L - 1) ||
      act < 0 || act > 1)
    return ZA_ERR_ARG;
  if (L < 1 || L > RC_MAX_TAPS) return ZA_ERR_UNSUPPORTED;
  const int tpb = 16;
  // (single tokens with a state to read: heads only)
  const int body = (n_tokens > n_seqs || L == 1) ? (n_tokens + tpb - 1) / tpb : 0;
  dim3 grid((C + 255) / 256, body + n_seqs), block(256);
#define ZA_CONV(T, TO)                                                                          \
  hipLaunchKernelGGL((causal_conv_silu_kernel<T, TO>), grid, block, 0, stream, (const T*)x,      \
                     x_stride, col0, taps, bias, state, slot_stride, token_seq, seq_start,       \
                     slot_id, (TO*)out, n_tokens, C, L, body, tpb, act)
  if (dtype == 0 && out_dtype == 0) ZA_CONV(float, float);
  else if (dtype == 1 && out_dtype == 0) ZA_CONV(bf16_t, float);
  else if (dtype == 1 && out_dtype == 1) ZA_CONV(bf16_t, bf16_t);
  else return ZA_ERR_UNSUPPORTED;
#undef ZA_CONV
  return za_launch_status();
}

extern "C" int za_causal_conv_silu(const void* x, int dtype, int x_stride, int col0,
                                   const float* taps, const float* bias, float* state,
                                   long long slot_stride, const int* token_seq,
                                   const int* seq_start, const int* slot_id, float* out,
                                   int n_tokens, int n_seqs, int C, int L, hipStream_t stream) {
  return za_causal_conv(x, dtype, x_stride, col0, taps, bias, state, slot_stride, token_seq,
                        seq_start, slot_id, out, 0, 1, n_tokens, n_seqs, C, L, stream);
}

// ------------------------------------------------------------------- recurrence
// What the two forms read, per token row t:
//   conv   [T][conv_width] 32-bit: the convolution's output.
//          SSD:   x of head h at x_col + h*dv, b of group g at k_col + g*dk, c at q_col + g*dk
//          delta: v of head h at x_col + h*dv (q and k come prepared, see below)
//   proj   [T][proj_stride] storage type (SSD): the raw step size of head h at gate_col + h
//   prep   [T][prep_width] 32-bit (delta), written by delta_prepare_kernel:
//          unit q of key head g at g*dk (times dk^-1/2), unit k at G*dk + g*dk, the decay of
//          head h and key channel i at 2*G*dk + h*dk + i, beta of head h at 2*G*dk + H*dk + h
struct RecurrenceArgs {
  const float* conv;
  int conv_width, q_col, k_col, x_col;
  const void* proj;
  int proj_stride, gate_col, proj_bf16;
  const float* prep;
  int prep_width;
  const float* dt_bias;   // SSD: [H]
  const float* A_log;     // SSD: [H]
  const float* D;         // SSD: [H]
  float* state;           // per slot [H][dv][dk]
  long long slot_stride;
  const int* seq_start;
  const int* slot_id;
  float* out;             // [T][H*dv] 32-bit
  int H, G, dk, dv;
  const float* fixed_decay;   // [H], or null: the SSD walk with this decay, dt = 1 and no
                              // raw step sizes (proj, dt_bias, A_log are not read then)
  const int* seq_count;       // [n], or null: the walkers' token counts, where their rows
                              // are given by (start, count) instead of n + 1 starts
};

// Everything of a token that does not depend on the state, for the delta rule: the unit
// vectors, the decays and the write strengths, once per token instead of once per
// workgroup that walks the token.  grid (tokens, jobs): the first 2*G jobs of a token make
// one unit vector each, the others take 256 decays each, the last one also the betas; a
// job is one trip to memory, and the jobs of a token run side by side.
template <typename T>
__global__ void __launch_bounds__(64)
delta_prepare_kernel(const float* __restrict__ conv, int conv_width, int q_col, int k_col,
                     const T* __restrict__ proj, int proj_stride, int gate_col,
                     const T* __restrict__ decay, int decay_stride,
                     const float* __restrict__ dt_bias, const float* __restrict__ A_log,
                     float* __restrict__ prep, int prep_width, int H, int G, int dk) {
  const int t = blockIdx.x, job = blockIdx.y, lane = threadIdx.x;
  float* row = prep + (size_t)t * prep_width;
  if (job < 2 * G) {
    const int is_k = job >= G, g = is_k ? job - G : job;
    const float* src = conv + (size_t)t * conv_width + (is_k ? k_col : q_col) + g * dk;
    float ss = 0.f;
    for (int i = lane; i < dk; i += 64) { const float v = src[i]; ss += v * v; }
    ss = wave_sum(ss);
    float scale = 1.0f / sqrtf(ss + 1e-6f);
    if (!is_k) scale *= 1.0f / sqrtf((float)dk);
    float* dst = row + (is_k ? G * dk : 0) + g * dk;
    for (int i = lane; i < dk; i += 64) dst[i] = src[i] * scale;
    return;
  }
  const int first = (job - 2 * G) * 256;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int idx = first + lane + 64 * k;
    if (idx < H * dk) {
      const float raw = to_f32<T>(decay[(size_t)t * decay_stride + idx]);
      row[2 * G * dk + idx] = expf(-expf(A_log[idx / dk]) * softplus_f(raw + dt_bias[idx]));
    }
  }
  if (job == (int)gridDim.y - 1)
    for (int h = lane; h < H; h += 64)
      row[2 * G * dk + H * dk + h] =
          sigmoid_f(to_f32<T>(proj[(size_t)t * proj_stride + gate_col + h]));
}

#define RC_ROWS 16   // state rows a lane keeps

// LDS index of key channel i when a lane owns RC_ROWS consecutive channels: four floats of
// padding per lane's share, so that a share starts on a 16-byte boundary (four-float
// reads) and the eight shares that eight neighbouring lanes read at once, 20 floats
// apart, cover the 32 banks once
#define RC_SHARE (RC_ROWS + 4)
__device__ __forceinline__ int lds_at(int i) { return i + (i / RC_ROWS) * 4; }

// The sum over the P neighbouring lanes (a power of two, the group starting at a multiple
// of P) that share a column; every lane of the group gets it.  Up to sixteen lanes the
// partners are reached with the vector unit's own lane patterns (pairs, quads, a half
// row and a row of sixteen mirrored), beyond that through the lane exchange.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false);
  return x + __builtin_bit_cast(float, moved);
}

template <int P>
__device__ __forceinline__ float group_sum(float x) {
  if (P >= 2) x = dpp_add<0xB1>(x);     // lanes 1 0 3 2 of every four
  if (P >= 4) x = dpp_add<0x4E>(x);     // lanes 2 3 0 1 of every four
  if (P >= 8) x = dpp_add<0x141>(x);    // a half row of eight, mirrored
  if (P >= 16) x = dpp_add<0x140>(x);   // a row of sixteen, mirrored
  if (P >= 32) x += __shfl_xor(x, 16, ZA_WAVE);
  if (P >= 64) x += __shfl_xor(x, 32, ZA_WAVE);
  return x;
}

// One wave a workgroup: 64 / P columns of one head's state, P lanes a column, RC_ROWS rows
// a lane.  The vectors of the next CH tokens are requested into registers while the
// current CH tokens are walked out of LDS, and put into the other LDS buffer afterwards.
// LONG: portions of many tokens (chunks of up to sixteen tokens, so that a chunk's walk
// outlasts the trip to memory of the next one's vectors); otherwise chunks as short as the
// load pattern allows, which leaves LDS for more waves when every portion is a token or two.
// (LONG == 1: half as long chunks, for steps with more waves than the chip has SIMDs, where
// LDS decides how many of them run at once)
template <int P, bool DELTA, int LONG>
__global__ void __launch_bounds__(64, 2)
matrix_recurrence_kernel(RecurrenceArgs a) {
  constexpr int R = RC_ROWS;
  constexpr int DKMAX = R * P;
  constexpr int CH_MIN = 4 * P < 64 ? 64 / (4 * P) : 1;
  constexpr int CH_LONG = (P <= 8 ? 16 : (P == 16 ? 8 : (P == 32 ? 4 : 2))) / (LONG == 1 ? 2 : 1);
  constexpr int CH = LONG ? (CH_LONG < CH_MIN ? CH_MIN : CH_LONG) : (CH_MIN < 2 ? 2 : CH_MIN);
  constexpr int NV = DELTA ? 3 : 2;                 // vectors of dk floats a token
  constexpr int KPAD = RC_SHARE * P;
  // a chunk's vectors come four floats a lane and load: LPV lanes cover a vector (or a
  // quarter of a long one), so one load instruction of the wave brings TPL tokens' worth
  constexpr int LPV = 4 * P < 64 ? 4 * P : 64;
  constexpr int TPL = 64 / LPV;
  constexpr int PIECES = DKMAX > 256 ? DKMAX / 256 : 1;
  constexpr int NLOAD = NV * (CH / TPL) * PIECES;    // four-float loads a lane and chunk
  __shared__ __attribute__((aligned(16))) float vecs[2][CH][NV][KPAD];
  __shared__ float scal[2][CH][2];                   // SSD: (decay, dt); delta: (beta, -)

  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int dk = a.dk, dv = a.dv;
  const int g = h / (a.H / a.G);
  const int col = blockIdx.z * (64 / P) + lane / P, part = lane % P;
  const bool owner = col < dv;
  const int start = a.seq_start[s];
  const int n = a.seq_count ? a.seq_count[s] : a.seq_start[s + 1] - start;

  // where the token's vectors lie: vector v of token t starts at base[v] + t * stride
  const float* base[NV];
  int stride;
  if (DELTA) {
    stride = a.prep_width;
    base[0] = a.prep + a.G * dk + g * dk;            // k
    base[1] = a.prep + g * dk;                       // q
    base[NV - 1] = a.prep + 2 * a.G * dk + h * dk;   // decays
  } else {
    stride = a.conv_width;
    base[0] = a.conv + a.k_col + g * dk;
    base[1] = a.conv + a.q_col + g * dk;
  }
  const float* xsrc = a.conv + a.x_col + h * dv + (owner ? col : 0);

  float* st = a.state + (size_t)a.slot_id[s] * a.slot_stride + ((size_t)h * dv + col) * dk + part * R;
  const bool vec_state = (dk % 4 == 0) && (a.slot_stride % 4 == 0) &&
                         ((reinterpret_cast<uintptr_t>(a.state) & 15) == 0);
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = 0.f;
  if (owner) {
    if (vec_state) {
#pragma unroll
      for (int r = 0; r < R; r += 4)
        if (part * R + r < dk) {
          const float4 v = *reinterpret_cast<const float4*>(st + r);
          S[r] = v.x; S[r + 1] = v.y; S[r + 2] = v.z; S[r + 3] = v.w;
        }
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (part * R + r < dk) S[r] = st[r];
    }
  }
  const bool fixed = !DELTA && a.fixed_decay != nullptr;
  const float fixed_a = fixed ? a.fixed_decay[h] : 0.f;
  const float neg_A = (DELTA || fixed) ? 0.f : -expf(a.A_log[h]);
  const float Dh = (DELTA || !a.D) ? 0.f : a.D[h];
  const float dtb = (DELTA || fixed) ? 0.f : a.dt_bias[h];

  // (whole four-float loads need the vectors to start on 16-byte boundaries)
  bool vec_loads = dk % 4 == 0 && stride % 4 == 0;
#pragma unroll
  for (int v = 0; v < NV; ++v)
    vec_loads = vec_loads && (reinterpret_cast<uintptr_t>(base[v]) & 15) == 0;
  const int lane_tt = lane / LPV, lane_i = (lane % LPV) * 4;
  float4 regs[NLOAD];
  float xnext[CH], snext = 0.f;
  int chunk_left = 0;       // tokens of the portion from the requested chunk's start on
  auto request = [&](int c0) {
#pragma unroll
    for (int j = 0; j < NLOAD; ++j) {
      const int v = j % NV, piece = (j / NV) % PIECES, group = j / (NV * PIECES);
      const int tt = group * TPL + lane_tt, i = piece * 256 + lane_i;
      // (a chunk's places beyond the portion's end hold tokens that change nothing: no
      // decay, nothing written, nothing read; the walk then needs no conditions)
      const float idle = (DELTA && v == NV - 1 && c0 + tt >= n) ? 1.f : 0.f;
      float4 x = make_float4(idle, idle, idle, idle);
      if (c0 + tt < n && i < dk) {
        const float* src = base[v] + (size_t)(start + c0 + tt) * stride + i;
        if (vec_loads) {
          x = *reinterpret_cast<const float4*>(src);
        } else {
          x.x = src[0];
          if (i + 1 < dk) x.y = src[1];
          if (i + 2 < dk) x.z = src[2];
          if (i + 3 < dk) x.w = src[3];
        }
      }
      regs[j] = x;
    }
#pragma unroll
    for (int tt = 0; tt < CH; ++tt)
      xnext[tt] = c0 + tt < n ? xsrc[(size_t)(start + c0 + tt) * a.conv_width] : 0.f;
    snext = 0.f;
    chunk_left = n - c0;
    if (lane < CH && c0 + lane < n) {
      const size_t t = start + c0 + lane;
      if (DELTA) {
        snext = a.prep[t * a.prep_width + 2 * a.G * dk + a.H * dk + h];
      } else if (!fixed) {
        const size_t at = t * a.proj_stride + a.gate_col + h;
        snext = a.proj_bf16 ? (float)((const bf16_t*)a.proj)[at] : ((const float*)a.proj)[at];
      }
    }
  };
  auto deposit = [&](int buf) {
#pragma unroll
    for (int j = 0; j < NLOAD; ++j) {
      const int v = j % NV, piece = (j / NV) % PIECES, group = j / (NV * PIECES);
      // (four channels from a multiple of four lie in one lane's share: side by side)
      *reinterpret_cast<float4*>(&vecs[buf][group * TPL + lane_tt][v][lds_at(piece * 256 + lane_i)]) =
          regs[j];
    }
    if (lane < CH) {
      if (DELTA) {
        scal[buf][lane][0] = snext;
      } else {
        const float dt = fixed ? 1.f : softplus_f(snext + dtb);
        scal[buf][lane][0] = lane < chunk_left ? (fixed ? fixed_a : expf(neg_A * dt)) : 1.f;
        scal[buf][lane][1] = lane < chunk_left ? dt : 0.f;
      }
    }
  };

  float xcur[CH];
  request(0);
  deposit(0);
#pragma unroll
  for (int tt = 0; tt < CH; ++tt) xcur[tt] = xnext[tt];
  __syncthreads();
  for (int c0 = 0, buf = 0; c0 < n; c0 += CH, buf ^= 1) {
    const bool more = c0 + CH < n;
    if (more) request(c0 + CH);
    const int cn = n - c0 < CH ? n - c0 : CH;
    float result[CH];      // stored after the walk: a store among the requests would make
                           // the walk wait for everything requested before it
#pragma unroll
    for (int tt = 0; tt < CH; ++tt) {
      {
        float kk[R], qq[R];
#pragma unroll
        for (int r = 0; r < R; r += 4) {
          const float4 k4 = *reinterpret_cast<const float4*>(&vecs[buf][tt][0][part * RC_SHARE + r]);
          const float4 q4 = *reinterpret_cast<const float4*>(&vecs[buf][tt][1][part * RC_SHARE + r]);
          kk[r] = k4.x; kk[r + 1] = k4.y; kk[r + 2] = k4.z; kk[r + 3] = k4.w;
          qq[r] = q4.x; qq[r + 1] = q4.y; qq[r + 2] = q4.z; qq[r + 3] = q4.w;
        }
        const float xv = xcur[tt];
        float o;
        if (DELTA) {
          float gg[R];
#pragma unroll
          for (int r = 0; r < R; r += 4) {
            const float4 g4 =
                *reinterpret_cast<const float4*>(&vecs[buf][tt][NV - 1][part * RC_SHARE + r]);
            gg[r] = g4.x; gg[r + 1] = g4.y; gg[r + 2] = g4.z; gg[r + 3] = g4.w;
          }
          float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
          for (int r = 0; r < R; r += 4) {
            S[r] *= gg[r]; S[r + 1] *= gg[r + 1]; S[r + 2] *= gg[r + 2]; S[r + 3] *= gg[r + 3];
            d0 = fmaf(S[r], kk[r], d0);
            d1 = fmaf(S[r + 1], kk[r + 1], d1);
            d2 = fmaf(S[r + 2], kk[r + 2], d2);
            d3 = fmaf(S[r + 3], kk[r + 3], d3);
          }
          const float dot = group_sum<P>((d0 + d1) + (d2 + d3));
          const float u = scal[buf][tt][0] * (xv - dot);
          float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
          for (int r = 0; r < R; r += 4) {
            S[r] = fmaf(kk[r], u, S[r]);
            S[r + 1] = fmaf(kk[r + 1], u, S[r + 1]);
            S[r + 2] = fmaf(kk[r + 2], u, S[r + 2]);
            S[r + 3] = fmaf(kk[r + 3], u, S[r + 3]);
            a0 = fmaf(S[r], qq[r], a0);
            a1 = fmaf(S[r + 1], qq[r + 1], a1);
            a2 = fmaf(S[r + 2], qq[r + 2], a2);
            a3 = fmaf(S[r + 3], qq[r + 3], a3);
          }
          o = group_sum<P>((a0 + a1) + (a2 + a3));
        } else {
          const float decay_t = scal[buf][tt][0], dtx = scal[buf][tt][1] * xv;
          float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
          for (int r = 0; r < R; r += 4) {
            S[r] = fmaf(decay_t, S[r], dtx * kk[r]);
            S[r + 1] = fmaf(decay_t, S[r + 1], dtx * kk[r + 1]);
            S[r + 2] = fmaf(decay_t, S[r + 2], dtx * kk[r + 2]);
            S[r + 3] = fmaf(decay_t, S[r + 3], dtx * kk[r + 3]);
            a0 = fmaf(S[r], qq[r], a0);
            a1 = fmaf(S[r + 1], qq[r + 1], a1);
            a2 = fmaf(S[r + 2], qq[r + 2], a2);
            a3 = fmaf(S[r + 3], qq[r + 3], a3);
          }
          o = fmaf(Dh, xv, group_sum<P>((a0 + a1) + (a2 + a3)));
        }
        result[tt] = o;
      }
    }
    if (part == 0 && owner) {
#pragma unroll
      for (int tt = 0; tt < CH; ++tt)
        if (tt < cn) a.out[(size_t)(start + c0 + tt) * a.H * dv + h * dv + col] = result[tt];
    }
    if (more) {
      deposit(buf ^ 1);
#pragma unroll
      for (int tt = 0; tt < CH; ++tt) xcur[tt] = xnext[tt];
    }
    __syncthreads();
  }
  if (owner) {
    if (vec_state) {
#pragma unroll
      for (int r = 0; r < R; r += 4)
        if (part * R + r < dk)
          *reinterpret_cast<float4*>(st + r) = make_float4(S[r], S[r + 1], S[r + 2], S[r + 3]);
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (part * R + r < dk) st[r] = S[r];
    }
  }
}

template <bool DELTA>
static int launch_recurrence(const RecurrenceArgs& a, int n_seqs, int P, bool long_portions,
                             hipStream_t stream) {
  dim3 grid(n_seqs, a.H, (a.dv * P + 63) / 64), block(64);
  // more waves than SIMDs (256 compute units of four): shorter chunks, more waves at once
  const bool crowded = (long long)grid.x * grid.y * grid.z > 1024;
#define ZA_RECURRENCE(PP)                                                                      \
  case PP:                                                                                     \
    if (long_portions && crowded)                                                              \
      hipLaunchKernelGGL((matrix_recurrence_kernel<PP, DELTA, 1>), grid, block, 0, stream, a); \
    else if (long_portions)                                                                    \
      hipLaunchKernelGGL((matrix_recurrence_kernel<PP, DELTA, 2>), grid, block, 0, stream, a); \
    else                                                                                       \
      hipLaunchKernelGGL((matrix_recurrence_kernel<PP, DELTA, 0>), grid, block, 0, stream, a); \
    break
  switch (P) {
    ZA_RECURRENCE(1);
    ZA_RECURRENCE(2);
    ZA_RECURRENCE(4);
    ZA_RECURRENCE(8);
    ZA_RECURRENCE(16);
    ZA_RECURRENCE(32);
    ZA_RECURRENCE(64);
    default: return ZA_ERR_UNSUPPORTED;
  }
#undef ZA_RECURRENCE
  return za_launch_status();
}

// `form`: 0 = SSD, 1 = gated delta rule, 2 = fixed decay (`decay` then holds H 32-bit
// decays, one per head; proj, dt_bias, A_log and D are not read).  `lanes` (P): the power of two, at most 64, with
// 16 * P >= dk that splits a column's rows.  `prep` (delta): [n_tokens][prep_width]
// floats of scratch, prep_width >= 2*G*dk + H*dk + H.
extern "C" int za_matrix_recurrence(int form, int dtype, const float* conv, int conv_width,
                                    int q_col, int k_col, int x_col, const void* proj,
                                    int proj_stride, int gate_col, const void* decay,
                                    int decay_stride, const float* dt_bias, const float* A_log,
                                    const float* D, float* prep, int prep_width, float* state,
                                    long long slot_stride, const int* seq_start,
                                    const int* slot_id, float* out, int n_tokens, int n_seqs,
                                    int H, int G, int dk, int dv, int lanes,
                                    hipStream_t stream) {
  if (n_seqs == 0 || n_tokens == 0) return 0;
  if (form < 0 || form > 2) return ZA_ERR_ARG;
  if (n_seqs < 0 || n_tokens < 0 || H <= 0 || G <= 0 || H % G || dk <= 0 || dv <= 0 || !conv ||
      !state || !seq_start || !slot_id || !out)
    return ZA_ERR_ARG;
  if (form != 2 && (!proj || !dt_bias || !A_log)) return ZA_ERR_ARG;
  if (form == 2 && !decay) return ZA_ERR_ARG;
  if (form == 0 && !D) return ZA_ERR_ARG;
  if (form == 1 && (!decay || decay_stride < H * dk || !prep ||
                    prep_width < 2 * G * dk + H * dk + H))
    return ZA_ERR_ARG;
  if (lanes < 1 || lanes > 64 || (lanes & (lanes - 1)) || lanes * RC_ROWS < dk ||
      slot_stride < (long long)H * dk * dv)
    return ZA_ERR_ARG;
  if (dtype != 0 && dtype != 1) return ZA_ERR_UNSUPPORTED;
  RecurrenceArgs a{conv, conv_width, q_col, k_col, x_col, proj, proj_stride, gate_col, dtype,
                   prep, prep_width, dt_bias, A_log, form == 2 ? nullptr : D, state, slot_stride,
                   seq_start, slot_id, out, H, G, dk, dv,
                   form == 2 ? (const float*)decay : nullptr, nullptr};
  // (a function of the step's shape alone, as a recorded step needs it)
  const bool long_portions = n_tokens > 4 * n_seqs;
  if (form != 1) return launch_recurrence<false>(a, n_seqs, lanes, long_portions, stream);
  const dim3 prep_grid(n_tokens, 2 * G + (H * dk + 255) / 256);
  if (dtype == 0)
    hipLaunchKernelGGL((delta_prepare_kernel<float>), prep_grid, dim3(64), 0, stream, conv,
                       conv_width, q_col, k_col, (const float*)proj, proj_stride, gate_col,
                       (const float*)decay, decay_stride, dt_bias, A_log, prep, prep_width, H, G,
                       dk);
  else
    hipLaunchKernelGGL((delta_prepare_kernel<bf16_t>), prep_grid, dim3(64), 0, stream, conv,
                       conv_width, q_col, k_col, (const bf16_t*)proj, proj_stride, gate_col,
                       (const bf16_t*)decay, decay_stride, dt_bias, A_log, prep, prep_width, H, G,
                       dk);
  const int rc = za_launch_status();
  if (rc != 0) return rc;
  return launch_recurrence<true>(a, n_seqs, lanes, long_portions, stream);
}

// ------------------------------------------------- fixed decay, long portions in chunks
// With a constant decay a head the state is linear in what the tokens bring, so a long
// portion need not be walked in one chain.  It is cut into chunks (the step's work items
// of CHUNK consecutive rows of one request):
//   1. every chunk is walked by itself from an empty state (matrix_recurrence_kernel with
//      one walker a chunk), leaving o_local[t] and its own final state L_c;
//   2. chunk_state_prefix: per request, in the order of its chunks, the state BEFORE chunk c,
//      B_c = B_(c-1) d^n(c-1) + L_(c-1), B_0 the request's carried state; the last one goes
//      back to the request's slot.  One thread a state element.
//   3. chunk_correct: o[t] = o_local[t] + d^(j+1) B_c^T q_t for token j of chunk c.
// All in 32-bit; powers of the decay as exp2(n log2 d).  A prompt of 2,048 tokens becomes
// eight chains of 256 tokens side by side instead of one of 2,048.
__global__ void __launch_bounds__(256)
chunk_state_prefix_kernel(float* __restrict__ chunk_state, float* __restrict__ state,
                          long long slot_stride, const int* __restrict__ slot_id,
                          const int* __restrict__ item_seq, const int* __restrict__ item_count,
                          int n_items, const float* __restrict__ decay, int elems, int per_head) {
  const int s = blockIdx.x;
  const int e = blockIdx.y * 256 + threadIdx.x;
  if (e >= elems) return;
  const float l2 = log2f(decay[e / per_head]);
  float* slot = state + (size_t)slot_id[s] * slot_stride + e;
  float S = *slot;
  for (int i = 0; i < n_items; ++i) {
    if (item_seq[i] != s) continue;
    float* at = chunk_state + (size_t)i * elems + e;
    const float local = *at;
    *at = S;
    const float a = decay[e / per_head] == 0.f ? 0.f : exp2f((float)item_count[i] * l2);
    S = fmaf(a, S, local);
  }
  *slot = S;
}

#define CC_TOKENS 16    // tokens whose queries are staged at a time
template <int DKR>      // rows of a state column kept in registers: dk <= DKR
__global__ void __launch_bounds__(128)
chunk_correct_kernel(const float* __restrict__ vectors, int width, int q_col,
                     const float* __restrict__ chunk_state, const int* __restrict__ item_row0,
                     const int* __restrict__ item_count, const float* __restrict__ decay,
                     float* __restrict__ out, int H, int dk, int dv, int tokens_per_block) {
  __shared__ float qs[CC_TOKENS][DKR];
  const int item = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int row0 = item_row0[item], cnt = item_count[item];
  const int t_begin = blockIdx.z * tokens_per_block;
  int t_end = t_begin + tokens_per_block;
  if (t_end > cnt) t_end = cnt;
  if (t_begin >= cnt) return;
  const float d = decay[h];
  const float l2 = log2f(d);
  const size_t elems = (size_t)H * dv * dk;
  for (int c0 = 0; c0 < dv; c0 += 128) {
    const int col = c0 + tid;
    float S[DKR];
#pragma unroll
    for (int r = 0; r < DKR; ++r) S[r] = 0.f;
    if (col < dv) {
      const float* src = chunk_state + (size_t)item * elems + ((size_t)h * dv + col) * dk;
#pragma unroll
      for (int r = 0; r < DKR; ++r)
        if (r < dk) S[r] = src[r];
    }
    for (int tb = t_begin; tb < t_end; tb += CC_TOKENS) {
      __syncthreads();
      // (rows beyond dk and tokens beyond the block's end are zeros: every product below
      // runs over all DKR rows)
      for (int idx = tid; idx < CC_TOKENS * DKR; idx += 128) {
        const int tt = idx / DKR, r = idx % DKR;
        qs[tt][r] = (r < dk && tb + tt < t_end)
                        ? vectors[(size_t)(row0 + tb + tt) * width + q_col + h * dk + r] : 0.f;
      }
      __syncthreads();
      if (col < dv) {
        // what the tokens' read-outs hold is requested for all of them before the first
        // product, and four sums run side by side in each
        float* o = out + (size_t)(row0 + tb) * H * dv + h * dv + col;
        float old[CC_TOKENS];
#pragma unroll
        for (int tt = 0; tt < CC_TOKENS; ++tt)
          old[tt] = tb + tt < t_end ? o[(size_t)tt * H * dv] : 0.f;
#pragma unroll
        for (int tt = 0; tt < CC_TOKENS; ++tt) {
          float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
          for (int r = 0; r < DKR; r += 4) {
            d0 = fmaf(S[r], qs[tt][r], d0);
            d1 = fmaf(S[r + 1], qs[tt][r + 1], d1);
            d2 = fmaf(S[r + 2], qs[tt][r + 2], d2);
            d3 = fmaf(S[r + 3], qs[tt][r + 3], d3);
          }
          const float w = d == 0.f ? 0.f : exp2f((float)(tb + tt + 1) * l2);
          if (tb + tt < t_end) o[(size_t)tt * H * dv] = fmaf(w, (d0 + d1) + (d2 + d3), old[tt]);
        }
      }
    }
  }
}

// `vectors` as retention_prepare leaves them; `item_*`: the step's work items of at most
// `chunk` rows (n_items of them; with n_items == n_seqs the plain walk does the same); `iota`:
// 0 .. n_items - 1; `chunk_state`: n_items * H*dv*dk floats, zero on entry.
extern "C" int za_retention_chunked(const float* vectors, int width, int q_col, int k_col,
                                    int x_col, const float* decay, float* state,
                                    long long slot_stride, const int* slot_id,
                                    const int* item_seq, const int* item_row0,
                                    const int* item_count, const int* iota, int n_items,
                                    int n_seqs, int chunk, float* chunk_state, float* out,
                                    int n_tokens, int H, int dk, int dv, int lanes,
                                    hipStream_t stream) {
  if (n_tokens == 0 || n_items == 0) return 0;
  if (n_tokens < 0 || n_items < n_seqs || n_seqs <= 0 || chunk <= 0 || H <= 0 || dk <= 0 || dv <= 0 ||
      !vectors || !decay || !state || !slot_id || !item_seq || !item_row0 || !item_count ||
      !iota || !chunk_state || !out)
    return ZA_ERR_ARG;
  if (dk > 128) return ZA_ERR_UNSUPPORTED;
  if (lanes < 1 || lanes > 64 || (lanes & (lanes - 1)) || lanes * RC_ROWS < dk ||
      slot_stride < (long long)H * dk * dv)
    return ZA_ERR_ARG;
  const long long elems = (long long)H * dk * dv;
  RecurrenceArgs a{vectors, width, q_col, k_col, x_col, nullptr, 0, 0, 0, nullptr, 0, nullptr,
                   nullptr, nullptr, chunk_state, elems, item_row0, iota, out, H, H, dk, dv,
                   decay, item_count};
  int rc = launch_recurrence<false>(a, n_items, lanes, n_tokens > 4 * n_items, stream);
  if (rc != 0) return rc;
  hipLaunchKernelGGL(chunk_state_prefix_kernel, dim3(n_seqs, (unsigned)((elems + 255) / 256)),
                     dim3(256), 0, stream, chunk_state, state, slot_stride, slot_id, item_seq,
                     item_count, n_items, decay, (int)elems, dk * dv);
  rc = za_launch_status();
  if (rc != 0) return rc;
  const int tokens_per_block = 64;      // an item has at most `chunk` rows
  dim3 grid(n_items, H, (unsigned)((chunk + tokens_per_block - 1) / tokens_per_block));
  if (dk <= 64)
    hipLaunchKernelGGL((chunk_correct_kernel<64>), grid, dim3(128), 0, stream, vectors, width,
                       q_col, chunk_state, item_row0, item_count, decay, out, H, dk, dv,
                       tokens_per_block);
  else
    hipLaunchKernelGGL((chunk_correct_kernel<128>), grid, dim3(128), 0, stream, vectors, width,
                       q_col, chunk_state, item_row0, item_count, decay, out, H, dk, dv,
                       tokens_per_block);
  return za_launch_status();
}

// ------------------------------------------------------------ retention's vectors
// What the fixed-decay walk reads, from the opening projection's rows: per token the
// queries and keys of every head with the first `rot` elements of each rotated by the
// token's position (element i paired with i + rot/2, angle = position * inv_freq[i]) and
// the keys times `k_scale`, then the values, all as 32-bit floats:
//   prep[t] = [q: H*dk | k: H*dk | v: H*dv]
// grid (tokens, heads), one wave.
template <typename T>
__global__ void __launch_bounds__(64)
retention_prepare_kernel(const T* __restrict__ proj, int proj_stride, int q_col, int k_col,
                         int v_col, const int* __restrict__ positions,
                         const float* __restrict__ inv_freq, float* __restrict__ prep, int H,
                         int dk, int dv, int rot, float k_scale, int act) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const T* row = proj + (size_t)t * proj_stride;
  float* dst = prep + (size_t)t * (2 * H * dk + H * dv);
  const int pos = positions[t], half = rot / 2;
  for (int i = lane; i < dk; i += 64) {
    // (`act` 1: silu on what the projection gave, before anything else)
    float q = to_f32<T>(row[q_col + h * dk + i]);
    float k = to_f32<T>(row[k_col + h * dk + i]);
    if (act) { q = silu_f(q); k = silu_f(k); }
    float qo = q, ko = k;
    if (i < rot) {
      const bool low = i < half;
      const int j = low ? i : i - half, partner = low ? i + half : i - half;
      float cs, sn;
      rope_angle(pos, inv_freq[j], &cs, &sn);
      float qp = to_f32<T>(row[q_col + h * dk + partner]);
      float kp = to_f32<T>(row[k_col + h * dk + partner]);
      if (act) { qp = silu_f(qp); kp = silu_f(kp); }
      qo = low ? rope_rotate_low(q, qp, cs, sn) : rope_rotate_high(q, qp, cs, sn);
      ko = low ? rope_rotate_low(k, kp, cs, sn) : rope_rotate_high(k, kp, cs, sn);
    }
    dst[h * dk + i] = qo;
    dst[H * dk + h * dk + i] = ko * k_scale;
  }
  for (int i = lane; i < dv; i += 64) {
    const float v = to_f32<T>(row[v_col + h * dv + i]);
    dst[2 * H * dk + h * dv + i] = act ? silu_f(v) : v;
  }
}

extern "C" int za_retention_prepare_act(const void* proj, int dtype, int proj_stride, int q_col,
                                    int k_col, int v_col, const int* positions,
                                    const float* inv_freq, float* prep, int n_tokens, int H, int dk,
                                    int dv, int rot, float k_scale, int act, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || H <= 0 || dk <= 0 || dv <= 0 || !proj || !positions || !prep || rot < 0 ||
      rot > dk || rot % 2 || (rot > 0 && !inv_freq) || q_col < 0 || k_col < 0 || v_col < 0 ||
      act < 0 || act > 1 || q_col + H * dk > proj_stride || k_col + H * dk > proj_stride ||
      v_col + H * dv > proj_stride)
    return ZA_ERR_ARG;
  dim3 grid(n_tokens, H), block(64);
  if (dtype == 0)
    hipLaunchKernelGGL((retention_prepare_kernel<float>), grid, block, 0, stream,
                       (const float*)proj, proj_stride, q_col, k_col, v_col, positions, inv_freq,
                       prep, H, dk, dv, rot, k_scale, act);
  else if (dtype == 1)
    hipLaunchKernelGGL((retention_prepare_kernel<bf16_t>), grid, block, 0, stream,
                       (const bf16_t*)proj, proj_stride, q_col, k_col, v_col, positions, inv_freq,
                       prep, H, dk, dv, rot, k_scale, act);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}

extern "C" int za_retention_prepare(const void* proj, int dtype, int proj_stride, int q_col,
                                    int k_col, int v_col, const int* positions,
                                    const float* inv_freq, float* prep, int n_tokens, int H, int dk,
                                    int dv, int rot, float k_scale, hipStream_t stream) {
  return za_retention_prepare_act(proj, dtype, proj_stride, q_col, k_col, v_col, positions,
                                  inv_freq, prep, n_tokens, H, dk, dv, rot, k_scale, 0, stream);
}

// ------------------------------------------------------------- gated group norm
// grid (tokens, groups); a workgroup reduces one group of `group` columns.
#define GN_VPT 16   // values a thread keeps between the sum of squares and the scaling
template <typename T>
__global__ void __launch_bounds__(256)
gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ gate, int gate_stride,
                        int gate_col, const float* __restrict__ w, int wlen, T* __restrict__ out,
                        int out_stride, int out_col, int width, int group, float eps, int silu_gate,
                        int gate_first, float out_scale) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, c0 = blockIdx.y * group;
  const float* yr = y + (size_t)t * width + c0;
  const T* gr = gate + (size_t)t * gate_stride + gate_col + c0;
  T* o = out + (size_t)t * out_stride + out_col + c0;
  const int bd = blockDim.x;
  float ss = 0.f;
  if (group <= bd * GN_VPT) {
    // one trip to memory: every load is requested before anything is summed
    float v[GN_VPT], act[GN_VPT], wv[GN_VPT];
#pragma unroll
    for (int k = 0; k < GN_VPT; ++k) {
      const int i = threadIdx.x + k * bd;
      v[k] = i < group ? yr[i] : 0.f;
      act[k] = i < group ? to_f32<T>(gr[i]) : 0.f;
      wv[k] = i < group ? w[(c0 + i) % wlen] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < GN_VPT; ++k) {
      act[k] = silu_gate ? silu_f(act[k]) : sigmoid_f(act[k]);
      if (gate_first) v[k] *= act[k];
      ss += v[k] * v[k];
    }
    ss = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(ss / (float)group + eps);
#pragma unroll
    for (int k = 0; k < GN_VPT; ++k) {
      const int i = threadIdx.x + k * bd;
      float r = v[k] * scale * wv[k];
      if (!gate_first) r *= act[k];
      if (i < group) o[i] = from_f32<T>(r * out_scale);
    }
    return;
  }
  for (int i = threadIdx.x; i < group; i += bd) {
    float v = yr[i];
    if (gate_first) {
      const float gv = to_f32<T>(gr[i]);
      v *= silu_gate ? silu_f(gv) : sigmoid_f(gv);
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)group + eps);
  for (int i = threadIdx.x; i < group; i += bd) {
    const float gv = to_f32<T>(gr[i]);
    const float act = silu_gate ? silu_f(gv) : sigmoid_f(gv);
    float v = yr[i];
    if (gate_first) v *= act;
    v = v * scale * w[(c0 + i) % wlen];
    if (!gate_first) v *= act;
    o[i] = from_f32<T>(v * out_scale);
  }
}

// The same for groups of at most 256 columns (a head's width): a wave a group, four
// groups a workgroup, the group's values in registers, the sum over the wave's lanes
// alone (no barrier).  grid: ceil(tokens * groups / 4).
template <typename T>
__global__ void __launch_bounds__(256)
gated_group_norm_wave_kernel(const float* __restrict__ y, const T* __restrict__ gate,
                             int gate_stride, int gate_col, const float* __restrict__ w, int wlen,
                             T* __restrict__ out, int out_stride, int out_col, int width, int group,
                             float eps, int silu_gate, int gate_first, float out_scale,
                             long long n_groups_total) {
  const int lane = threadIdx.x & 63;
  const long long gi = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (gi >= n_groups_total) return;
  const int per_token = width / group;
  const size_t t = (size_t)(gi / per_token);
  const int c0 = (int)(gi % per_token) * group;
  const float* yr = y + t * width + c0;
  const T* gr = gate + t * gate_stride + gate_col + c0;
  T* o = out + t * out_stride + out_col + c0;
  float v[4], act[4], wv[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int i = lane + 64 * k;
    v[k] = i < group ? yr[i] : 0.f;
    act[k] = i < group ? to_f32<T>(gr[i]) : 0.f;
    wv[k] = i < group ? w[(c0 + i) % wlen] : 0.f;
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    act[k] = silu_gate ? silu_f(act[k]) : sigmoid_f(act[k]);
    if (gate_first) v[k] *= act[k];
    ss += v[k] * v[k];
  }
  ss = wave_sum(ss);
  const float scale = 1.0f / sqrtf(ss / (float)group + eps);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int i = lane + 64 * k;
    float r = v[k] * scale * wv[k];
    if (!gate_first) r *= act[k];
    if (i < group) o[i] = from_f32<T>(r * out_scale);
  }
}

extern "C" int za_gated_group_norm(const float* y, const void* gate, int dtype, int gate_stride,
                                   int gate_col, const float* w, int wlen, void* out,
                                   int out_stride, int out_col, int n_tokens, int width, int group,
                                   float eps, int silu_gate, int gate_first, float out_scale,
                                   hipStream_t stream) {
  if (n_tokens == 0) return 0;
  if (n_tokens < 0 || width <= 0 || group <= 0 || width % group || !y || !gate || !w || !out ||
      wlen <= 0 || gate_col < 0 || gate_col + width > gate_stride || out_col < 0 ||
      out_col + width > out_stride)
    return ZA_ERR_ARG;
  if (group <= 256 && dtype >= 0 && dtype <= 1) {
    // small groups (a head each): a wave a group
    const long long total = (long long)n_tokens * (width / group);
    dim3 wgrid((unsigned)((total + 3) / 4)), wblock(256);
    if (dtype == 0)
      hipLaunchKernelGGL((gated_group_norm_wave_kernel<float>), wgrid, wblock, 0, stream, y,
                         (const float*)gate, gate_stride, gate_col, w, wlen, (float*)out, out_stride,
                         out_col, width, group, eps, silu_gate, gate_first, out_scale, total);
    else
      hipLaunchKernelGGL((gated_group_norm_wave_kernel<bf16_t>), wgrid, wblock, 0, stream, y,
                         (const bf16_t*)gate, gate_stride, gate_col, w, wlen, (bf16_t*)out,
                         out_stride, out_col, width, group, eps, silu_gate, gate_first, out_scale,
                         total);
    return za_launch_status();
  }
  dim3 grid(n_tokens, width / group), block(group <= 64 ? 64 : (group <= 128 ? 128 : 256));
  if (dtype == 0)
    hipLaunchKernelGGL((gated_group_norm_kernel<float>), grid, block, 0, stream, y,
                       (const float*)gate, gate_stride, gate_col, w, wlen, (float*)out, out_stride,
                       out_col, width, group, eps, silu_gate, gate_first, out_scale);
  else if (dtype == 1)
    hipLaunchKernelGGL((gated_group_norm_kernel<bf16_t>), grid, block, 0, stream, y,
                       (const bf16_t*)gate, gate_stride, gate_col, w, wlen, (bf16_t*)out,
                       out_stride, out_col, width, group, eps, silu_gate, gate_first, out_scale);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}
