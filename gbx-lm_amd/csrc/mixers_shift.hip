// Stream kernels of sandwich-norm layers (a norm in front of and behind every sublayer) and what sits around them:
//
//   embed_pair_kernel            token embedding + hashed (previous token, token) pair embedding; the previous token of a step's first
//                                row is state of the sequence.
//   norm_shift_kernel            RMS norm of a stream row and of the row before it, h = n + (n_prev - n) * shift; the norm of a
//                                sequence's last row is left in its slot for the next step.
//   branch_norm_add_norm_kernel  x += rms_norm(branch) * w (the branch optionally a weighted sum of candidate rows plus a row every
//                                token takes), then the next sublayer's norm of the new x.
//   normed_pair_mean_kernel      half the sum of two separately normed rows.
//   gate_mul_kernel              act(gate) * up over rows that are not neighbours in memory.
//
// One workgroup per row; statistics in fp32 with a fixed summation order: a row's result does not depend on which other rows share the
// step, and the norm a row's successor recomputes for its shift has the bits the row itself left in the slot.
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256, NW = NT / 64;
constexpr int ZR = 16;             // values a thread keeps between a statistic and its use (rows up to ZR * NT wide; wider rows re-read)

template <typename T>
__global__ __launch_bounds__(NT) void embed_pair_kernel(const T* __restrict__ table, const T* __restrict__ pair, const int64_t* __restrict__ tokens,
                                                       int64_t* __restrict__ state, const int* __restrict__ seq, const int* __restrict__ tok,
                                                       float* __restrict__ x, int width, int64_t buckets, int64_t mul_prev, int64_t mul_cur) {
  const int64_t t = blockIdx.x;
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], n = seq[4 * b + 2], row0 = seq[4 * b + 3];
  const int64_t token = tokens[t];
  const bool first_of_step = pos == pos0;
  // unconditional loads from addresses that exist (a step's first row has no row before it in the step: it reads itself)
  const int64_t before = tokens[first_of_step ? t : t - 1];
  const int64_t kept = state[slot];
  const int64_t prev = first_of_step ? kept : before;
  const int64_t row = pos == 0 ? buckets : (prev * mul_prev + token * mul_cur) % buckets;
  const T* e = table + token * width;
  const T* p = pair + row * width;
  for (int c = threadIdx.x; c < width; c += NT) x[t * width + c] = to_f32(e[c]) + to_f32(p[c]);
  if (first_of_step) {
    __syncthreads();                       // every thread has read the slot
    if (threadIdx.x == 0) state[slot] = tokens[row0 + n - 1];
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void norm_shift_kernel(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ shift,
                                                       float* __restrict__ state, const int* __restrict__ seq, const int* __restrict__ tok,
                                                       T* __restrict__ h, int width, float eps) {
  __shared__ float red[NW];
  const int64_t t = blockIdx.x;
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], n = seq[4 * b + 2], row0 = seq[4 * b + 3];
  const bool first_of_step = pos == pos0;
  const float* xc = x + t * width;
  const float* xp = x + (first_of_step ? t : t - 1) * width;         // the row before, where the step holds it
  float sc = 0.f, sp = 0.f;
  for (int c = threadIdx.x; c < width; c += NT) {
    const float a = xc[c], q = xp[c];
    sc += a * a;
    sp += q * q;
  }
  sc = block_sum<NW>(sc, red);
  sp = block_sum<NW>(sp, red);
  const float rc = 1.f / sqrtf(sc / width + eps), rp = 1.f / sqrtf(sp / width + eps);
  float* st = state + static_cast<int64_t>(slot) * width;
  float rl = rc;
  const float* xl = xc;
  if (first_of_step && n > 1) {            // this workgroup also leaves the sequence's last norm in the slot: it is the one that read it
    xl = x + static_cast<int64_t>(row0 + n - 1) * width;
    float sl = 0.f;
    for (int c = threadIdx.x; c < width; c += NT) { const float a = xl[c]; sl += a * a; }
    sl = block_sum<NW>(sl, red);
    rl = 1.f / sqrtf(sl / width + eps);
  }
  for (int c = threadIdx.x; c < width; c += NT) {
    const float wc = w[c];
    const float cur = xc[c] * rc * wc;
    const float kept = st[c];
    const float prev = first_of_step ? (pos0 > 0 ? kept : 0.f) : xp[c] * rp * wc;
    h[t * width + c] = from_f32<T>(cur + (prev - cur) * shift[c]);
    if (first_of_step) st[c] = xl[c] * rl * wc;
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void branch_norm_add_norm_kernel(float* __restrict__ x, const T* __restrict__ branch, const float* __restrict__ mix,
                                                                 const T* __restrict__ extra, const float* __restrict__ w,
                                                                 const float* __restrict__ next_w, T* __restrict__ h, int width, int top, float eps) {
  __shared__ float red[NW];
  __shared__ float ml[64];
  const int64_t t = blockIdx.x;
  const T* b = branch + t * top * width;
  const T* ex = extra ? extra + t * width : nullptr;
  const bool mixed = mix != nullptr;
  if (mixed && threadIdx.x < min(top, 64)) ml[threadIdx.x] = mix[t * top + threadIdx.x];
  __syncthreads();
  auto z_at = [&](int c) {
    float z;
    if (!mixed) z = to_f32(b[c]);
    else {
      z = 0.f;
      for (int s = 0; s < top; ++s) z += (s < 64 ? ml[s] : mix[t * top + s]) * to_f32(b[s * width + c]);
    }
    if (ex) z += to_f32(ex[c]);
    return z;
  };
  float zr[ZR];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < ZR; ++i) {
    const int c = threadIdx.x + i * NT;
    zr[i] = c < width ? z_at(c) : 0.f;
    ss += zr[i] * zr[i];
  }
  for (int c = threadIdx.x + ZR * NT; c < width; c += NT) { const float z = z_at(c); ss += z * z; }
  ss = block_sum<NW>(ss, red);
  const float r = 1.f / sqrtf(ss / width + eps);
  float* xr = x + t * width;
  float s2 = 0.f;
#pragma unroll
  for (int i = 0; i < ZR; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < width) {
      const float v = xr[c] + zr[i] * r * w[c];
      xr[c] = v;
      zr[i] = v;
      s2 += v * v;
    }
  }
  for (int c = threadIdx.x + ZR * NT; c < width; c += NT) {
    const float v = xr[c] + z_at(c) * r * w[c];
    xr[c] = v;
    s2 += v * v;
  }
  if (!next_w) return;
  s2 = block_sum<NW>(s2, red);
  const float r2 = 1.f / sqrtf(s2 / width + eps);
#pragma unroll
  for (int i = 0; i < ZR; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < width) h[t * width + c] = from_f32<T>(zr[i] * r2 * next_w[c]);
  }
  for (int c = threadIdx.x + ZR * NT; c < width; c += NT) h[t * width + c] = from_f32<T>(xr[c] * r2 * next_w[c]);      // (a thread re-reads what it wrote)
}

template <typename T>
__global__ __launch_bounds__(NT) void normed_pair_mean_kernel(const T* __restrict__ a, const T* __restrict__ b, const float* __restrict__ wa,
                                                             const float* __restrict__ wb, T* __restrict__ out, int width, float eps) {
  __shared__ float red[NW];
  const int64_t t = blockIdx.x;
  const T* ar = a + t * width;
  const T* br = b + t * width;
  float sa = 0.f, sb = 0.f;
  for (int c = threadIdx.x; c < width; c += NT) {
    const float u = to_f32(ar[c]), v = to_f32(br[c]);
    sa += u * u;
    sb += v * v;
  }
  sa = block_sum<NW>(sa, red);
  sb = block_sum<NW>(sb, red);
  const float ra = 1.f / sqrtf(sa / width + eps), rb = 1.f / sqrtf(sb / width + eps);
  for (int c = threadIdx.x; c < width; c += NT)
    out[t * width + c] = from_f32<T>(0.5f * (to_f32(ar[c]) * ra * wa[c] + to_f32(br[c]) * rb * wb[c]));
}

template <typename T, bool FAST>
__global__ __launch_bounds__(NT) void gate_mul_kernel(const T* __restrict__ gate, int64_t gate_stride, const T* __restrict__ up, int64_t up_stride,
                                                     T* __restrict__ out, int F, int kind) {
  const int64_t t = blockIdx.y;
  const T* g = gate + t * gate_stride;
  const T* u = up + t * up_stride;
  for (int f = blockIdx.x * NT + threadIdx.x; f < F; f += gridDim.x * NT)
    out[t * F + f] = from_f32<T>(glu_act<FAST>(to_f32(g[f]), to_f32(u[f]), kind, 0.f, 0.f));
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

int gbxm_embed_hashed_pair(const void* table, const void* pair, const int64_t* tokens, int64_t* state, const int32_t* seq, const int32_t* tok,
                           float* x, int64_t T_, int32_t width, int64_t buckets, int64_t mul_prev, int64_t mul_cur, int32_t act, void* stream) {
  if (!act_ok(act) || !table || !pair || !tokens || !state || !seq || !tok || !x || width <= 0 || buckets < 1 || mul_prev < 0 || mul_cur < 0 || T_ < 0)
    return fail(GBXM_ERR_INVALID, "embed_hashed_pair: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (embed_pair_kernel<T><<<dim3(T_), NT, 0, s>>>(static_cast<const T*>(table), static_cast<const T*>(pair), tokens, state, seq, tok, x,
                                                                     width, buckets, mul_prev, mul_cur)));
  return after_launch("embed_hashed_pair");
}

int gbxm_norm_token_shift(const float* x, const float* w, const float* shift, float* state, const int32_t* seq, const int32_t* tok, void* h,
                          int64_t T_, int32_t width, float eps, int32_t act, void* stream) {
  if (!act_ok(act) || !x || !w || !shift || !state || !seq || !tok || !h || width <= 0 || T_ < 0)
    return fail(GBXM_ERR_INVALID, "norm_token_shift: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (norm_shift_kernel<T><<<dim3(T_), NT, 0, s>>>(x, w, shift, state, seq, tok, static_cast<T*>(h), width, eps)));
  return after_launch("norm_token_shift");
}

int gbxm_branch_norm_add_norm(float* x, const void* branch, const float* mix, const void* extra, const float* w, const float* next_w, void* h,
                              int64_t T_, int32_t width, int32_t top, float eps, int32_t act, void* stream) {
  if (!act_ok(act) || !x || !branch || !w || width <= 0 || top < 1 || T_ < 0 || (top > 1 && !mix) || (next_w && !h))
    return fail(GBXM_ERR_INVALID, "branch_norm_add_norm: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (branch_norm_add_norm_kernel<T><<<dim3(T_), NT, 0, s>>>(x, static_cast<const T*>(branch), mix, static_cast<const T*>(extra), w,
                                                                               next_w, static_cast<T*>(h), width, top, eps)));
  return after_launch("branch_norm_add_norm");
}

int gbxm_normed_pair_mean(const void* a, const void* b, const float* wa, const float* wb, void* out, int64_t T_, int32_t width, float eps,
                          int32_t act, void* stream) {
  if (!act_ok(act) || !a || !b || !wa || !wb || !out || width <= 0 || T_ < 0) return fail(GBXM_ERR_INVALID, "normed_pair_mean: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (normed_pair_mean_kernel<T><<<dim3(T_), NT, 0, s>>>(static_cast<const T*>(a), static_cast<const T*>(b), wa, wb,
                                                                           static_cast<T*>(out), width, eps)));
  return after_launch("normed_pair_mean");
}

int gbxm_gate_mul(const void* gate, int64_t gate_stride, const void* up, int64_t up_stride, void* out, int64_t T_, int32_t F, int32_t kind,
                  int32_t act, void* stream) {
  if (!act_ok(act) || !gate || !up || !out || F <= 0 || gate_stride < F || up_stride < F || T_ < 0 ||
      (kind != GBXM_GLU_SILU && kind != GBXM_GLU_GELU_TANH && kind != GBXM_GLU_SIGMOID))
    return fail(GBXM_ERR_INVALID, "gate_mul: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t el = act == GBXM_BF16 ? 2 : 4;
  for (int64_t t0 = 0; t0 < T_; t0 += 65535) {          // rows ride on grid.y: long steps go in slices
    const int64_t n = T_ - t0 < 65535 ? T_ - t0 : 65535;
    const dim3 grid(min((F + NT - 1) / NT, 64), n);
    const char* g = static_cast<const char*>(gate) + t0 * gate_stride * el;
    const char* u = static_cast<const char*>(up) + t0 * up_stride * el;
    char* o = static_cast<char*>(out) + t0 * F * el;
    if (act == GBXM_BF16)
      gate_mul_kernel<bf16_t, true><<<grid, NT, 0, s>>>(reinterpret_cast<const bf16_t*>(g), gate_stride, reinterpret_cast<const bf16_t*>(u), up_stride,
                                                        reinterpret_cast<bf16_t*>(o), F, kind);
    else
      gate_mul_kernel<float, false><<<grid, NT, 0, s>>>(reinterpret_cast<const float*>(g), gate_stride, reinterpret_cast<const float*>(u), up_stride,
                                                        reinterpret_cast<float*>(o), F, kind);
  }
  return after_launch("gate_mul");
}

}  // extern "C"
