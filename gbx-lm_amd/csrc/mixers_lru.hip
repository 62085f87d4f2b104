// A recurrent block around a gated linear recurrent unit: a diagonal recurrence per channel whose decay and input gate come from
// block-diagonal products of the convolved input.
//
//   causal_conv_rows_kernel    short causal convolution over time per channel with a bias, fp32 out; inputs before the step come from
//                              the slot's tail, zeros before the sequence.
//   block_gate_logits_kernel   the two gates' block-diagonal products for steps of few rows: workgroups per (row, block, share of the
//                              output rows), the block's inputs in LDS, a wave per output row of the matrix (lanes across the inputs,
//                              16-byte loads), fp32 sums in a fixed order.  (Prompt-sized steps take a batched fp32 matrix product of the vendor library.)
//   gated_lru_scan_kernel      a = exp(-rate sigmoid(r) softplus(lam)), S <- a S + sqrt(1 - a^2) sigmoid(i) u, out = S gelu(y).  A workgroup
//                              owns CB channels of one sequence and walks its rows in chunks of CH tokens: all threads form (a, input)
//                              of the chunk in parallel into LDS, CB threads run the recurrence over the chunk (two LDS reads and one
//                              multiply-add per token, operands read eight tokens ahead), all threads form the product with the gelu
//                              branch.  All of the next chunk's operands are loaded while the recurrence runs.
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256, NW = NT / 64;

template <typename T>
__global__ __launch_bounds__(NT) void causal_conv_rows_kernel(const T* __restrict__ x, int64_t x_stride, const T* __restrict__ conv,
                                                             const float* __restrict__ bias, const T* __restrict__ tail, const int* __restrict__ seq,
                                                             const int* __restrict__ tok, float* __restrict__ out, int C, int taps) {
  const int64_t t = blockIdx.x;
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], row0 = seq[4 * b + 3];
  const int keep = taps - 1;
  const T* tl = tail ? tail + static_cast<int64_t>(slot) * keep * C : nullptr;
  for (int c = blockIdx.y * NT + threadIdx.x; c < C; c += gridDim.y * NT) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int src = pos - keep + j;
      float v = 0.f;
      if (src >= pos0) v = to_f32(x[(row0 + (src - pos0)) * x_stride + c]);
      else if (src >= 0) v = to_f32(tl[static_cast<int64_t>(src - pos0 + keep) * C + c]);
      acc += to_f32(conv[c * taps + j]) * v;
    }
    out[t * C + c] = bias ? acc + bias[c] : acc;
  }
}

// grid (rows, blocks, splits of the block's output rows).  LDS: the block's bs inputs.  A wave owns one output row at a time, lanes
// across its inputs with 16-byte loads where the block size allows; the splits spread a step of few rows over the chip.
template <typename T>
__global__ __launch_bounds__(NT) void block_gate_logits_kernel(const float* __restrict__ u, const T* __restrict__ w, const float* __restrict__ bias,
                                                              float* __restrict__ logits, int blocks, int bs, int n_out) {
  extern __shared__ float ub[];
  const int64_t t = blockIdx.x;
  const int b = blockIdx.y;
  const float* ur = u + (t * blocks + b) * bs;
  for (int i = threadIdx.x; i < bs; i += NT) ub[i] = ur[i];
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* wb = w + static_cast<int64_t>(b) * n_out * bs;
  float* lr = logits + (t * blocks + b) * n_out;
  constexpr int PER = 16 / sizeof(T);
  const bool vec = bs % PER == 0;                  // rows then start 16-byte aligned
  for (int o = blockIdx.z * NW + wave; o < n_out; o += gridDim.z * NW) {
    const T* wr = wb + static_cast<int64_t>(o) * bs;
    float s = 0.f;
    if (vec) {
      for (int i = lane * PER; i < bs; i += 64 * PER) {
        T v[PER];
        *reinterpret_cast<uint4*>(v) = *reinterpret_cast<const uint4*>(wr + i);
#pragma unroll
        for (int j = 0; j < PER; ++j) s += to_f32(v[j]) * ub[i + j];
      }
    } else {
      for (int i = lane; i < bs; i += 64) s += to_f32(wr[i]) * ub[i];
    }
    s = wave_sum(s);
    if (lane == 0) lr[o] = s + bias[b * n_out + o];
  }
}

constexpr int CB = 16;             // channels of a workgroup
constexpr int CH = 64;             // tokens of a chunk
constexpr int PER = CB * CH / NT;  // elements of a chunk per thread

template <bool FAST> __device__ __forceinline__ float gelu_tanh_(float z) {
  return 0.5f * z * (1.f + tanh_<FAST>(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// grid (ceil(C / CB), B).  logits rows [t][block][2 bs] with strides in floats (a batched product leaves them block-major).
template <typename T, bool FAST>
__global__ __launch_bounds__(NT) void gated_lru_scan_kernel(const float* __restrict__ u, const float* __restrict__ logits, int64_t lg_t, int64_t lg_b,
                                                           const float* __restrict__ lam_sp, const T* __restrict__ y, int64_t y_stride,
                                                           float* __restrict__ state, T* __restrict__ out, const int* __restrict__ seq, int C, int bs,
                                                           float rate) {
  __shared__ float a_l[CH][CB + 1];
  __shared__ float in_l[CH][CB + 1];       // the input term, then the state after the token
  const int b = blockIdx.y;
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], n = seq[4 * b + 2], row0 = seq[4 * b + 3];
  const int c0 = blockIdx.x * CB;
  const int cl = threadIdx.x % CB, tl0 = threadIdx.x / CB;          // this thread's channel of the tile and its first token of a chunk
  const int c = c0 + cl;
  const bool live = c < C;
  const int cc = live ? c : C - 1;
  const int blk = cc / bs, ci = cc - blk * bs;
  const float sp = lam_sp[cc];
  float* st = state + static_cast<int64_t>(slot) * C;
  float S = 0.f;
  if (threadIdx.x < CB) { S = st[cc]; S = pos0 > 0 ? S : 0.f; }
  float lr[PER], li[PER], uu[PER];
  T yy[PER];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int tt = min(t0 + tl0 + k * (NT / CB), n - 1);
      const int64_t row = row0 + tt;
      const float* lp = logits + row * lg_t + static_cast<int64_t>(blk) * lg_b;
      lr[k] = lp[ci];
      li[k] = lp[bs + ci];
      uu[k] = u[row * C + cc];
      yy[k] = y[row * y_stride + cc];
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < n; t0 += CH) {
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int tt = tl0 + k * (NT / CB);
      const float r = sigmoid_<FAST>(lr[k]), ig = sigmoid_<FAST>(li[k]);
      const float a = exp_<FAST>(-rate * r * sp);
      a_l[tt][cl] = a;
      in_l[tt][cl] = sqrtf(fmaxf(1.f - a * a, 0.f)) * (ig * uu[k]);
    }
    float g[PER];                                   // the other branch of this chunk, before its operands are replaced by the next chunk's
#pragma unroll
    for (int k = 0; k < PER; ++k) g[k] = gelu_tanh_<FAST>(to_f32(yy[k]));
    __syncthreads();
    if (t0 + CH < n) fetch(t0 + CH);
    const int cn = min(CH, n - t0);
    if (threadIdx.x < CB) {
      // eight tokens' operands are read before the eight dependent multiply-adds (LDS latency once per eight, not per token)
      for (int t8 = 0; t8 < cn; t8 += 8) {
        float a8[8], i8[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) { a8[j] = a_l[t8 + j][cl]; i8[j] = in_l[t8 + j][cl]; }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (t8 + j < cn) S = a8[j] * S + i8[j];
          i8[j] = S;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) in_l[t8 + j][cl] = i8[j];
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int tt = tl0 + k * (NT / CB);
      if (tt < cn && live) {
        const int64_t row = row0 + t0 + tt;
        out[row * C + c] = from_f32<T>(in_l[tt][cl] * g[k]);
      }
    }
    __syncthreads();
  }
  if (threadIdx.x < CB && live) st[c] = S;
}

// Steps in which every sequence brings one row: a thread per (sequence, channel), the same arithmetic in the same order.
template <typename T, bool FAST>
__global__ __launch_bounds__(NT) void gated_lru_step_kernel(const float* __restrict__ u, const float* __restrict__ logits, int64_t lg_t, int64_t lg_b,
                                                           const float* __restrict__ lam_sp, const T* __restrict__ y, int64_t y_stride,
                                                           float* __restrict__ state, T* __restrict__ out, const int* __restrict__ seq, int C, int bs,
                                                           float rate) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * NT + threadIdx.x;
  if (c >= C) return;
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1];
  const int64_t row = seq[4 * b + 3];
  const int blk = c / bs, ci = c - blk * bs;
  const float* lp = logits + row * lg_t + static_cast<int64_t>(blk) * lg_b;
  const float lr = lp[ci], li = lp[bs + ci], uu = u[row * C + c], sp = lam_sp[c];
  const float yv = to_f32(y[row * y_stride + c]);
  float* st = state + static_cast<int64_t>(slot) * C + c;
  float S = *st;
  S = pos0 > 0 ? S : 0.f;
  const float r = sigmoid_<FAST>(lr), ig = sigmoid_<FAST>(li);
  const float a = exp_<FAST>(-rate * r * sp);
  const float in = sqrtf(fmaxf(1.f - a * a, 0.f)) * (ig * uu);
  S = a * S + in;
  *st = S;
  out[row * C + c] = from_f32<T>(S * gelu_tanh_<FAST>(yv));
}

bool act_ok(int act) { return act == GBXM_BF16 || act == GBXM_F32; }

}  // namespace
}  // namespace gbxm

using namespace gbxm;

#define GBXM_DISPATCH(act, CALL)              \
  do {                                        \
    if ((act) == GBXM_BF16) { using T = bf16_t; CALL; } else { using T = float; CALL; } \
  } while (0)

extern "C" {

int gbxm_causal_conv_rows(const void* x, int64_t x_stride, const void* conv, const float* bias, const void* tail, const int32_t* seq,
                          const int32_t* tok, float* out, int64_t T_, int32_t C, int32_t taps, int32_t act, void* stream) {
  if (!act_ok(act) || !x || !conv || !seq || !tok || !out || C < 1 || taps < 1 || (taps > 1 && !tail) || x_stride < C || T_ < 0)
    return fail(GBXM_ERR_INVALID, "causal_conv_rows: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int64_t splits = (1024 + T_ - 1) / T_;                 // a step of few rows spreads a row's channels over workgroups
  const int64_t most = (C + NT - 1) / NT;
  if (splits > most) splits = most;
  const dim3 grid(T_, static_cast<unsigned>(splits < 1 ? 1 : splits));
  GBXM_DISPATCH(act, (causal_conv_rows_kernel<T><<<grid, NT, 0, s>>>(static_cast<const T*>(x), x_stride, static_cast<const T*>(conv), bias,
                                                                       static_cast<const T*>(tail), seq, tok, out, C, taps)));
  return after_launch("causal_conv_rows");
}

int gbxm_block_gate_logits(const float* u, const void* w, const float* bias, float* logits, int64_t T_, int32_t blocks, int32_t bs, int32_t n_out,
                           int32_t act, void* stream) {
  if (!act_ok(act) || !u || !w || !bias || !logits || blocks < 1 || bs < 1 || n_out < 1 || T_ < 0)
    return fail(GBXM_ERR_INVALID, "block_gate_logits: bad argument");
  if (blocks > 65535) return fail(GBXM_ERR_UNSUPPORTED, "block_gate_logits: more than 65535 blocks");
  if (bs > 12288) return fail(GBXM_ERR_UNSUPPORTED, "block_gate_logits: blocks of %d channels (at most 12288)", bs);
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int64_t splits = (512 + T_ * blocks - 1) / (T_ * blocks);      // enough workgroups for the chip, a wave keeps at least one output row
  const int64_t most = (n_out + NW - 1) / NW;
  if (splits > most) splits = most;
  if (splits < 1) splits = 1;
  GBXM_DISPATCH(act, (block_gate_logits_kernel<T><<<dim3(T_, blocks, static_cast<unsigned>(splits)), NT, bs * sizeof(float), s>>>(
                         u, static_cast<const T*>(w), bias, logits, blocks, bs, n_out)));
  return after_launch("block_gate_logits");
}

int gbxm_gated_lru_scan(const float* u, const float* logits, int64_t lg_t, int64_t lg_b, const float* lam_sp, const void* y, int64_t y_stride,
                        float* state, void* out, const int32_t* seq, int32_t B, int64_t T_, int32_t C, int32_t bs, float rate, int32_t act,
                        void* stream) {
  if (!act_ok(act) || !u || !logits || !lam_sp || !y || !state || !out || !seq || B < 0 || T_ < 0 || C < 1 || bs < 1 || C % bs || y_stride < C)
    return fail(GBXM_ERR_INVALID, "gated_lru_scan: bad argument");
  if (B == 0 || T_ == 0) return GBXM_OK;
  if (B > 65535) return fail(GBXM_ERR_UNSUPPORTED, "gated_lru_scan: more than 65535 sequences in a step");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (T_ == B) {                                   // every sequence brings one row
    const dim3 sgrid((C + NT - 1) / NT, B);
    if (act == GBXM_BF16)
      gated_lru_step_kernel<bf16_t, false><<<sgrid, NT, 0, s>>>(u, logits, lg_t, lg_b, lam_sp, static_cast<const bf16_t*>(y), y_stride, state,
                                                              static_cast<bf16_t*>(out), seq, C, bs, rate);
    else
      gated_lru_step_kernel<float, false><<<sgrid, NT, 0, s>>>(u, logits, lg_t, lg_b, lam_sp, static_cast<const float*>(y), y_stride, state,
                                                             static_cast<float*>(out), seq, C, bs, rate);
    return after_launch("gated_lru_scan");
  }
  const dim3 grid((C + CB - 1) / CB, B);
  if (act == GBXM_BF16)
    gated_lru_scan_kernel<bf16_t, false><<<grid, NT, 0, s>>>(u, logits, lg_t, lg_b, lam_sp, static_cast<const bf16_t*>(y), y_stride, state,
                                                            static_cast<bf16_t*>(out), seq, C, bs, rate);
  else
    gated_lru_scan_kernel<float, false><<<grid, NT, 0, s>>>(u, logits, lg_t, lg_b, lam_sp, static_cast<const float*>(y), y_stride, state,
                                                           static_cast<float*>(out), seq, C, bs, rate);
  return after_launch("gated_lru_scan");
}

}  // extern "C"
