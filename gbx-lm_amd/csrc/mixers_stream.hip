// Several residual streams (one launch per sublayer boundary: stream mixing + write of the sublayer's output + read + layer norm),
// gated activations of feed-forwards, and the sigmoid router with a choice correction and expert groups.  One workgroup per row;
// statistics in fp32 with a fixed summation order, so a row's result does not depend on which other rows share the step.
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256, NW = NT / 64;
constexpr int MAXS = 8;           // streams
constexpr int UR = 8;             // read-out values a thread keeps between the passes (rows up to UR * NT wide; wider rows re-read)

// S is a template parameter and every load is issued from an address inside the row (channels past the row's end are clamped, their
// results dropped): loads under a run-time condition wait for one another, and a row would cost the sum of their latencies.
template <typename T, int S>
__global__ __launch_bounds__(NT) void hyper_step_kernel(float* __restrict__ X, const T* __restrict__ y, const float* __restrict__ y_mix,
                                                       const float* __restrict__ mix, const float* __restrict__ write, const float* __restrict__ read,
                                                       const float* __restrict__ norm_w, const float* __restrict__ norm_b, T* __restrict__ h,
                                                       float* __restrict__ out_u, int width, int top, float eps) {
  __shared__ float red[NW];
  __shared__ float sm[S * S + 2 * S];
  __shared__ float ml[64];
  extern __shared__ float ul[];            // [width] when width > UR * NT, else unused
  const int64_t t = blockIdx.x;
  float* xr = X + t * S * width;
  float* mixl = sm;
  float* wl = sm + S * S;
  float* rl = wl + S;
  const bool upd = y != nullptr;
  if (threadIdx.x < S * S) mixl[threadIdx.x] = upd ? mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    wl[threadIdx.x] = upd ? write[threadIdx.x] : 0.f;
    rl[threadIdx.x] = read ? read[threadIdx.x] : 1.f;
  }
  const bool mixed = y_mix != nullptr;
  if (upd && mixed && threadIdx.x < top) ml[threadIdx.x] = y_mix[t * top + threadIdx.x];
  __syncthreads();
  const T* yr = upd ? y + t * top * width : nullptr;
  const bool wide = width > UR * NT;
  float ur[UR];
  float sum = 0.f;
  // pass 1: the update of every channel's S values (a channel is independent of the others) and the read-out u
  auto channel = [&](int c) {
    const bool live = c < width;
    const int cc = live ? c : width - 1;
    float xs[S];
#pragma unroll
    for (int i = 0; i < S; ++i) xs[i] = xr[i * width + cc];
    float u = 0.f;
    if (upd) {
      float z;
      if (!mixed) z = to_f32(yr[cc]);
      else {
        z = 0.f;
        for (int k = 0; k < top; ++k) z += ml[k] * to_f32(yr[k * width + cc]);
      }
#pragma unroll
      for (int j = 0; j < S; ++j) {
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < S; ++i) v += mixl[i * S + j] * xs[i];
        v += wl[j] * z;
        if (live) xr[j * width + cc] = v;
        u += rl[j] * v;
      }
    } else {
#pragma unroll
      for (int j = 0; j < S; ++j) u += rl[j] * xs[j];
    }
    return live ? u : 0.f;
  };
#pragma unroll
  for (int i = 0; i < UR; ++i) {
    const int c = threadIdx.x + i * NT;
    ur[i] = channel(c);
    sum += ur[i];
    if (wide && c < width) ul[c] = ur[i];
  }
  for (int c = threadIdx.x + UR * NT; c < width; c += NT) { const float u = channel(c); ul[c] = u; sum += u; }
  if (!norm_w) {
#pragma unroll
    for (int i = 0; i < UR; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < width) out_u[t * width + c] = ur[i];
    }
    for (int c = threadIdx.x + UR * NT; c < width; c += NT) out_u[t * width + c] = ul[c];
    return;
  }
  const float mean = block_sum<NW>(sum, red) / width;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < UR; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < width) { const float d = ur[i] - mean; ss += d * d; }
  }
  for (int c = threadIdx.x + UR * NT; c < width; c += NT) { const float d = ul[c] - mean; ss += d * d; }
  const float r = 1.f / sqrtf(block_sum<NW>(ss, red) / width + eps);
#pragma unroll
  for (int i = 0; i < UR; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < width) h[t * width + c] = from_f32<T>((ur[i] - mean) * r * norm_w[c] + norm_b[c]);
  }
  for (int c = threadIdx.x + UR * NT; c < width; c += NT) h[t * width + c] = from_f32<T>((ul[c] - mean) * r * norm_w[c] + norm_b[c]);
}

template <typename T>
void launch_hyper_step(int S, dim3 grid, size_t lds, hipStream_t s, float* X, const void* y, const float* y_mix, const float* mix, const float* write,
                       const float* read, const float* norm_w, const float* norm_b, void* h, float* out_u, int width, int top, float eps) {
#define GBXM_HS(N) hyper_step_kernel<T, N><<<grid, NT, lds, s>>>(X, static_cast<const T*>(y), y_mix, mix, write, read, norm_w, norm_b, static_cast<T*>(h), \
                                                               out_u, width, top, eps)
  switch (S) {
    case 1: GBXM_HS(1); break;
    case 2: GBXM_HS(2); break;
    case 3: GBXM_HS(3); break;
    case 4: GBXM_HS(4); break;
    case 5: GBXM_HS(5); break;
    case 6: GBXM_HS(6); break;
    case 7: GBXM_HS(7); break;
    default: GBXM_HS(8); break;
  }
#undef GBXM_HS
}

template <typename T, bool FAST>
__global__ __launch_bounds__(NT) void glu_kernel(const T* __restrict__ gu, int64_t stride, T* __restrict__ out, int F, int kind, float limit,
                                                float alpha) {
  const int64_t t = blockIdx.y;
  const T* g = gu + t * stride;
  for (int f = blockIdx.x * NT + threadIdx.x; f < F; f += gridDim.x * NT)
    out[t * F + f] = from_f32<T>(glu_act<FAST>(to_f32(g[f]), to_f32(g[F + f]), kind, limit, alpha));
}

// One wave per row.  LDS: s [E], c [E] (choice scores; -inf once taken or outside the kept groups), group scores [n_groups].
__global__ __launch_bounds__(64) void route_sigmoid_groups_kernel(const float* __restrict__ logits, const float* __restrict__ correction,
                                                                 int* __restrict__ idx, float* __restrict__ weight, int E, int top, int n_groups,
                                                                 int keep_groups, int renorm, float scale) {
  extern __shared__ float lds[];
  float* sl = lds;
  float* cl = lds + E;
  float* gl = lds + 2 * E;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) {
    const float s = 1.f / (1.f + expf(-logits[t * E + e]));
    sl[e] = s;
    cl[e] = s + correction[e];
  }
  __syncthreads();
  // arg-max over n values of `v` (ties: the lower index); every lane gets the result
  auto arg_max = [&](const float* v, int n) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < n; e += 64)
      if (v[e] > bv || bi == 0x7fffffff) { bv = v[e]; bi = e; }          // ascending e per lane: the first of equals stays
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi))) { bv = ov; bi = oi; }
    }
    return bi;
  };
  if (n_groups > 0) {
    const int size = E / n_groups;
    for (int g = lane; g < n_groups; g += 64) {
      float a = -INFINITY, b = -INFINITY;          // the two largest
      for (int e = g * size; e < (g + 1) * size; ++e) {
        const float v = cl[e];
        if (v > a) { b = a; a = v; } else if (v > b) b = v;
      }
      gl[g] = size > 1 ? a + b : a;
    }
    __syncthreads();
    for (int k = 0; k < keep_groups; ++k) {
      const int g = arg_max(gl, n_groups);
      __syncthreads();
      if (lane == 0) gl[g] = -INFINITY;            // taken: -inf marks a kept group from here on (scores are finite)
      __syncthreads();
    }
    for (int e = lane; e < E; e += 64)
      if (gl[e / size] != -INFINITY) cl[e] = -INFINITY;
    __syncthreads();
  }
  float chosen = 0.f;
  for (int k = 0; k < top; ++k) {
    const int e = arg_max(cl, E);
    __syncthreads();
    chosen += sl[e];
    if (lane == 0) { idx[t * top + k] = e; weight[t * top + k] = sl[e]; cl[e] = -INFINITY; }
    __syncthreads();
  }
  const float mul = renorm ? scale / (chosen + 1e-20f) : scale;
  for (int k = lane; k < top; k += 64) weight[t * top + k] = sl[idx[t * top + k]] * mul;
}

bool act_ok(int act) { return act == GBXM_BF16 || act == GBXM_F32; }

}  // namespace
}  // namespace gbxm

using namespace gbxm;

extern "C" {

int gbxm_hyper_step(float* X, const void* y, const float* y_mix, const float* mix, const float* write, const float* read, const float* norm_w,
                    const float* norm_b, void* h, float* out_u, int64_t T_, int32_t S, int32_t width, int32_t top, float eps, int32_t act,
                    void* stream) {
  if (!act_ok(act) || !X || S < 1 || width <= 0 || T_ < 0 || top < 1 || (y && (!mix || !write)) || (top > 1 && !y_mix) ||
      (norm_w ? (!norm_b || !h) : !out_u))
    return fail(GBXM_ERR_INVALID, "hyper_step: bad argument");
  if (S > MAXS) return fail(GBXM_ERR_UNSUPPORTED, "hyper_step: more than %d streams", MAXS);
  if (top > 64) return fail(GBXM_ERR_UNSUPPORTED, "hyper_step: more than 64 candidates per row");
  const size_t lds = width > UR * NT ? static_cast<size_t>(width) * sizeof(float) : 0;
  if (lds > 60 * 1024) return fail(GBXM_ERR_UNSUPPORTED, "hyper_step: rows of %d channels", width);
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (act == GBXM_BF16) launch_hyper_step<bf16_t>(S, dim3(T_), lds, s, X, y, y_mix, mix, write, read, norm_w, norm_b, h, out_u, width, top, eps);
  else launch_hyper_step<float>(S, dim3(T_), lds, s, X, y, y_mix, mix, write, read, norm_w, norm_b, h, out_u, width, top, eps);
  return after_launch("hyper_step");
}

int gbxm_glu(const void* gu, int64_t gu_stride, void* out, int64_t T_, int32_t F, int32_t kind, float limit, float alpha, int32_t act, void* stream) {
  if (!act_ok(act) || !gu || !out || F <= 0 || gu_stride < 2 * F || T_ < 0 || kind < GBXM_GLU_SILU || kind > GBXM_GLU_SIGMOID)
    return fail(GBXM_ERR_INVALID, "glu: bad argument");
  if (T_ == 0) return GBXM_OK;
  if (T_ > 65535) {                       // rows ride on grid.y: long steps go in slices
    for (int64_t t0 = 0; t0 < T_; t0 += 65535) {
      const int64_t n = T_ - t0 < 65535 ? T_ - t0 : 65535;
      const size_t el = act == GBXM_BF16 ? 2 : 4;
      const int rc = gbxm_glu(static_cast<const char*>(gu) + t0 * gu_stride * el, gu_stride, static_cast<char*>(out) + t0 * F * el, n, F, kind, limit,
                              alpha, act, stream);
      if (rc) return rc;
    }
    return GBXM_OK;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(min((F + NT - 1) / NT, 64), T_);
  if (act == GBXM_BF16)
    glu_kernel<bf16_t, true><<<grid, NT, 0, s>>>(static_cast<const bf16_t*>(gu), gu_stride, static_cast<bf16_t*>(out), F, kind, limit, alpha);
  else
    glu_kernel<float, false><<<grid, NT, 0, s>>>(static_cast<const float*>(gu), gu_stride, static_cast<float*>(out), F, kind, limit, alpha);
  return after_launch("glu");
}

int gbxm_route_sigmoid_groups(const float* logits, const float* correction, int32_t* idx, float* weight, int64_t T_, int32_t E, int32_t top,
                              int32_t n_groups, int32_t keep_groups, int32_t renorm, float scale, void* stream) {
  if (!logits || !correction || !idx || !weight || E <= 0 || top < 1 || top > E || T_ < 0 || n_groups < 0 ||
      (n_groups > 0 && (E % n_groups || keep_groups < 1 || keep_groups > n_groups || top > keep_groups * (E / n_groups))))
    return fail(GBXM_ERR_INVALID, "route_sigmoid_groups: bad argument");
  if (E > 4096) return fail(GBXM_ERR_UNSUPPORTED, "route_sigmoid_groups: more than 4096 experts");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  route_sigmoid_groups_kernel<<<dim3(T_), 64, (2 * E + (n_groups > 0 ? n_groups : 1)) * sizeof(float), s>>>(logits, correction, idx, weight, E, top, n_groups,
                                                                                                          keep_groups, renorm, scale);
  return after_launch("route_sigmoid_groups");
}

}  // extern "C"
