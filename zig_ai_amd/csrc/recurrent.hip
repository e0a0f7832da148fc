// Mixers that carry a matrix state from token to token, for any mix of prompt
// portions and single decoded tokens in one launch.  Everything that enters a
// recurrence is 32-bit: the state, decays, step sizes, gates and unit norms.
//
// 1. causal_conv_silu: a depth-wise causal convolution over a request's own inputs
//    followed by silu,
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
//    A column of S never meets another column: a thread (or P neighbouring lanes that
//    split the rows) keeps one column in registers across all tokens of the portion,
//    reads it from the slot at the start and stores it at the end.  The slot holds S
//    turned round, [head][column][row], so that a lane's rows are consecutive floats.
//    The per-token vectors of a chunk of tokens are prepared by the whole workgroup
//    into LDS (norms, decays, gates), then the tokens are walked in order.
//
// 3. gated_group_norm: y * act(gate) and an RMS norm over equal groups of columns, the
//    gate before or after the norm:
//      gate first:  v = y * act(gate);  out = v / rms(v) * w
//      gate last:   out = y / rms(y) * w * act(gate)
#include <math.h>

#include "common.h"

#define RC_MAX_TAPS 8
#define RC_CHUNK 16          // tokens prepared into LDS at a time, at most

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
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_silu_kernel(const T* __restrict__ x, int x_stride, int col0,
                        const float* __restrict__ taps, const float* __restrict__ bias,
                        float* __restrict__ state, long long slot_stride,
                        const int* __restrict__ token_seq, const int* __restrict__ seq_start,
                        const int* __restrict__ slot_id, float* __restrict__ out, int n_tokens,
                        int C, int L, int body_blocks, int tokens_per_block) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  float w[RC_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < RC_MAX_TAPS; ++j) w[j] = j < L ? taps[(size_t)c * L + j] : 0.f;
  const float b = bias ? bias[c] : 0.f;
  if ((int)blockIdx.y < body_blocks) {
    const int t0 = blockIdx.y * tokens_per_block;
    for (int t = t0; t < t0 + tokens_per_block && t < n_tokens; ++t) {
      const int rel = t - seq_start[token_seq[t]];
      if (rel < L - 1) continue;
      float acc = b;
#pragma unroll
      for (int j = 0; j < RC_MAX_TAPS; ++j)
        if (j < L)
          acc = fmaf(w[j], to_f32<T>(x[(size_t)(t - (L - 1 - j)) * x_stride + col0 + c]), acc);
      out[(size_t)t * C + c] = silu_f(acc);
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
    out[(size_t)(start + i) * C + c] = silu_f(acc);
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

extern "C" int za_causal_conv_silu(const void* x, int dtype, int x_stride, int col0,
                                   const float* taps, const float* bias, float* state,
                                   long long slot_stride, const int* token_seq,
                                   const int* seq_start, const int* slot_id, float* out,
                                   int n_tokens, int n_seqs, int C, int L, hipStream_t stream) {
  if (n_tokens == 0 || n_seqs == 0) return 0;
  if (n_tokens < 0 || n_seqs < 0 || C <= 0 || !x || !taps || !state || !token_seq || !seq_start ||
      !slot_id || !out || col0 < 0 || col0 + C > x_stride || slot_stride < (long long)C * (L - 1))
    return ZA_ERR_ARG;
  if (L < 1 || L > RC_MAX_TAPS) return ZA_ERR_UNSUPPORTED;
  const int tpb = 8;
  // (single tokens with a state to read: heads only)
  const int body = (n_tokens > n_seqs || L == 1) ? (n_tokens + tpb - 1) / tpb : 0;
  dim3 grid((C + 255) / 256, body + n_seqs), block(256);
  if (dtype == 0)
    hipLaunchKernelGGL((causal_conv_silu_kernel<float>), grid, block, 0, stream, (const float*)x,
                       x_stride, col0, taps, bias, state, slot_stride, token_seq, seq_start,
                       slot_id, out, n_tokens, C, L, body, tpb);
  else if (dtype == 1)
    hipLaunchKernelGGL((causal_conv_silu_kernel<bf16_t>), grid, block, 0, stream,
                       (const bf16_t*)x, x_stride, col0, taps, bias, state, slot_stride, token_seq,
                       seq_start, slot_id, out, n_tokens, C, L, body, tpb);
  else
    return ZA_ERR_UNSUPPORTED;
  return za_launch_status();
}

// ------------------------------------------------------------------- recurrence
// What the two forms read, per token row t:
//   conv   [T][conv_width] 32-bit: the convolution's output.
//          SSD:   x of head h at x_col + h*dv, b of group g at k_col + g*dk, c at q_col + g*dk
//          delta: q of key head g at q_col + g*dk, k at k_col + g*dk, v of head h at x_col + h*dv
//   proj   [T][proj_stride] storage type: the opening projection's raw output.
//          SSD:   dt of head h at gate_col + h
//          delta: beta of head h at gate_col + h
//   decay  [T][decay_stride] storage type (delta only): the decay's raw value per head and key
//          channel, head h's at columns h*dk
struct RecurrenceArgs {
  const float* conv;
  int conv_width, q_col, k_col, x_col;
  const void* proj;
  int proj_stride, gate_col;
  const void* decay;
  int decay_stride;
  const float* dt_bias;   // SSD: [H]; delta: [H*dk]
  const float* A_log;     // [H]
  const float* D;         // SSD: [H]
  float* state;           // per slot [H][dv][dk]
  long long slot_stride;
  const int* seq_start;
  const int* slot_id;
  float* out;             // [T][H*dv] 32-bit
  int H, G, dk, dv, P;
  int cols_per_block;     // columns of S a workgroup keeps (grid.z covers dv)
  int chunk;              // tokens prepared into LDS at a time (what fits)
};

// LDS index of key channel i when a lane owns R consecutive channels: one float of
// padding per lane's share, so that the P lanes of a column meet different banks
template <int R> __device__ __forceinline__ int lds_at(int i) { return i + i / R; }

template <typename T, int R, bool DELTA>
__global__ void __launch_bounds__(512)
matrix_recurrence_kernel(RecurrenceArgs a) {
  extern __shared__ float lds[];
  const int s = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  const int P = a.P, dk = a.dk, dv = a.dv;
  const int g = h / (a.H / a.G);
  const int col = blockIdx.z * a.cols_per_block + tid / P, part = tid % P;
  const bool owner = tid / P < a.cols_per_block && col < dv;
  const int kpad = lds_at<R>(dk - 1) + 1;
  // LDS: per chunk token: kvec[kpad], qvec[kpad], (delta) gvec[kpad], xvec[dv], 2 scalars
  const int CH = a.chunk;
  float* Kc = lds;
  float* Qc = Kc + CH * kpad;
  float* Gc = Qc + CH * kpad;
  float* Xc = Gc + (DELTA ? CH * kpad : 0);
  float* Sc = Xc + CH * dv;                // [chunk][2]: SSD (decay, dt); delta (beta, -)

  const int start = a.seq_start[s], n = a.seq_start[s + 1] - start;
  float* st = a.state + (size_t)a.slot_id[s] * a.slot_stride + ((size_t)h * dv + col) * dk;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = part * R + r;
    S[r] = (owner && i < dk) ? st[i] : 0.f;
  }
  const float neg_A = -expf(a.A_log[h]);
  const float Dh = DELTA ? 0.f : a.D[h];
  const int lane = tid & 63, wave = tid >> 6, nwaves = (blockDim.x + 63) >> 6;
  const T* proj = (const T*)a.proj;
  const T* decay = (const T*)a.decay;

  for (int c0 = 0; c0 < n; c0 += CH) {
    const int cn = n - c0 < CH ? n - c0 : CH;
    __syncthreads();     // the chunk before has been walked
    if (DELTA) {
      // unit vectors: a wave takes (token, q or k) pairs in turn
      for (int job = wave; job < 2 * cn; job += nwaves) {
        const int tt = job >> 1, is_k = job & 1;
        const float* src = a.conv + (size_t)(start + c0 + tt) * a.conv_width +
                           (is_k ? a.k_col : a.q_col) + g * dk;
        float ss = 0.f;
        for (int i = lane; i < dk; i += 64) { const float v = src[i]; ss += v * v; }
        ss = wave_sum(ss);
        float scale = 1.0f / sqrtf(ss + 1e-6f);
        if (!is_k) scale *= 1.0f / sqrtf((float)dk);
        float* dst = (is_k ? Kc : Qc) + tt * kpad;
        for (int i = lane; i < dk; i += 64) dst[lds_at<R>(i)] = src[i] * scale;
      }
      for (int idx = tid; idx < cn * dk; idx += blockDim.x) {
        const int tt = idx / dk, i = idx % dk;
        const float raw = to_f32<T>(decay[(size_t)(start + c0 + tt) * a.decay_stride + h * dk + i]);
        Gc[tt * kpad + lds_at<R>(i)] = expf(neg_A * softplus_f(raw + a.dt_bias[h * dk + i]));
      }
      if (tid < cn)
        Sc[tid * 2] = sigmoid_f(to_f32<T>(proj[(size_t)(start + c0 + tid) * a.proj_stride +
                                               a.gate_col + h]));
    } else {
      for (int idx = tid; idx < cn * dk; idx += blockDim.x) {
        const int tt = idx / dk, i = idx % dk;
        const float* row = a.conv + (size_t)(start + c0 + tt) * a.conv_width;
        Kc[tt * kpad + lds_at<R>(i)] = row[a.k_col + g * dk + i];
        Qc[tt * kpad + lds_at<R>(i)] = row[a.q_col + g * dk + i];
      }
      if (tid < cn) {
        const float raw = to_f32<T>(proj[(size_t)(start + c0 + tid) * a.proj_stride +
                                         a.gate_col + h]);
        const float dt = softplus_f(raw + a.dt_bias[h]);
        Sc[tid * 2] = expf(neg_A * dt);
        Sc[tid * 2 + 1] = dt;
      }
    }
    for (int idx = tid; idx < cn * dv; idx += blockDim.x) {
      const int tt = idx / dv, j = idx % dv;
      Xc[tt * dv + j] = a.conv[(size_t)(start + c0 + tt) * a.conv_width + a.x_col + h * dv + j];
    }
    __syncthreads();
    if (!owner) continue;
    for (int tt = 0; tt < cn; ++tt) {
      const float* kk = Kc + tt * kpad + part * (R + 1);
      const float* qq = Qc + tt * kpad + part * (R + 1);
      const float xv = Xc[tt * dv + col];
      float o;
      if (DELTA) {
        const float* gg = Gc + tt * kpad + part * (R + 1);
        float dot = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (part * R + r < dk) {
            S[r] *= gg[r];
            dot = fmaf(S[r], kk[r], dot);
          }
        }
        for (int off = 1; off < P; off <<= 1) dot += __shfl_xor(dot, off, ZA_WAVE);
        const float u = Sc[tt * 2] * (xv - dot);
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (part * R + r < dk) {
            S[r] = fmaf(kk[r], u, S[r]);
            acc = fmaf(S[r], qq[r], acc);
          }
        }
        for (int off = 1; off < P; off <<= 1) acc += __shfl_xor(acc, off, ZA_WAVE);
        o = acc;
      } else {
        const float decay_t = Sc[tt * 2], dtx = Sc[tt * 2 + 1] * xv;
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (part * R + r < dk) {
            S[r] = fmaf(decay_t, S[r], dtx * kk[r]);
            acc = fmaf(S[r], qq[r], acc);
          }
        }
        for (int off = 1; off < P; off <<= 1) acc += __shfl_xor(acc, off, ZA_WAVE);
        o = fmaf(Dh, xv, acc);
      }
      if (part == 0) a.out[(size_t)(start + c0 + tt) * a.H * dv + h * dv + col] = o;
    }
  }
  if (owner) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = part * R + r;
      if (i < dk) st[i] = S[r];
    }
  }
}

template <typename T, bool DELTA>
static int launch_recurrence(RecurrenceArgs a, int n_seqs, int R, hipStream_t stream) {
  const int threads = (a.cols_per_block * a.P + 63) / 64 * 64;
  const int kpad = a.dk + (a.dk - 1) / R + 1;
  const size_t per_token = sizeof(float) * ((size_t)kpad * (DELTA ? 3 : 2) + a.dv + 2);
  a.chunk = RC_CHUNK;
  while (a.chunk > 1 && a.chunk * per_token > 64 * 1024) a.chunk /= 2;
  const size_t lds = a.chunk * per_token;
  if (lds > 64 * 1024) return ZA_ERR_UNSUPPORTED;
  dim3 grid(n_seqs, a.H, (a.dv + a.cols_per_block - 1) / a.cols_per_block), block(threads);
#define ZA_RECURRENCE(RR)                                                                    \
  hipLaunchKernelGGL((matrix_recurrence_kernel<T, RR, DELTA>), grid, block, lds, stream, a)
  if (R == 8) ZA_RECURRENCE(8);
  else if (R == 16) ZA_RECURRENCE(16);
  else if (R == 32) ZA_RECURRENCE(32);
  else return ZA_ERR_UNSUPPORTED;
#undef ZA_RECURRENCE
  return za_launch_status();
}

// `form`: 0 = SSD, 1 = gated delta rule.  `lanes` (P): a power of two up to 64 that
// splits a column's dk rows; `rows_per_lane` (R): 8, 16 or 32 with R * P >= dk;
// `cols_per_block` columns of S (times P lanes, at most 512 threads) a workgroup.
extern "C" int za_matrix_recurrence(int form, int dtype, const float* conv, int conv_width,
                                    int q_col, int k_col, int x_col, const void* proj,
                                    int proj_stride, int gate_col, const void* decay,
                                    int decay_stride, const float* dt_bias, const float* A_log, const float* D,
                                    float* state, long long slot_stride, const int* seq_start,
                                    const int* slot_id, float* out, int n_seqs, int H, int G,
                                    int dk, int dv, int lanes, int rows_per_lane,
                                    int cols_per_block, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  if (n_seqs < 0 || H <= 0 || G <= 0 || H % G || dk <= 0 || dv <= 0 || !conv || !proj ||
      !dt_bias || !A_log || !state || !seq_start || !slot_id || !out)
    return ZA_ERR_ARG;
  if (form == 0 ? !D : (!decay || decay_stride < H * dk)) return ZA_ERR_ARG;
  if (lanes < 1 || lanes > 64 || (lanes & (lanes - 1)) || lanes * rows_per_lane < dk ||
      cols_per_block < 1 || cols_per_block * lanes > 512 ||
      slot_stride < (long long)H * dk * dv)
    return ZA_ERR_ARG;
  RecurrenceArgs a{conv, conv_width, q_col, k_col, x_col, proj, proj_stride, gate_col, decay,
                   decay_stride, dt_bias, A_log, D, state, slot_stride, seq_start, slot_id, out,
                   H, G, dk, dv, lanes, cols_per_block, RC_CHUNK};
  if (dtype == 0)
    return form ? launch_recurrence<float, true>(a, n_seqs, rows_per_lane, stream)
                : launch_recurrence<float, false>(a, n_seqs, rows_per_lane, stream);
  if (dtype == 1)
    return form ? launch_recurrence<bf16_t, true>(a, n_seqs, rows_per_lane, stream)
                : launch_recurrence<bf16_t, false>(a, n_seqs, rows_per_lane, stream);
  return ZA_ERR_UNSUPPORTED;
}

// ------------------------------------------------------------- gated group norm
// grid (tokens, groups); a workgroup reduces one group of `group` columns.
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
  float ss = 0.f;
  for (int i = threadIdx.x; i < group; i += blockDim.x) {
    float v = yr[i];
    if (gate_first) {
      const float gv = to_f32<T>(gr[i]);
      v *= silu_gate ? silu_f(gv) : sigmoid_f(gv);
    }
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(ss / (float)group + eps);
  T* o = out + (size_t)t * out_stride + out_col + c0;
  for (int i = threadIdx.x; i < group; i += blockDim.x) {
    const float gv = to_f32<T>(gr[i]);
    const float act = silu_gate ? silu_f(gv) : sigmoid_f(gv);
    float v = yr[i];
    if (gate_first) v *= act;
    v = v * scale * w[(c0 + i) % wlen];
    if (!gate_first) v *= act;
    o[i] = from_f32<T>(v * out_scale);
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
