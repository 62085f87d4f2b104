// Routed gated MLPs over dense stacked experts:  y[t][s] = down_e (silu(gate_e h_t) * (up_e h_t)),  e = idx[t][s].
//
//   * row kernels -- weight-bandwidth bound: the kernels of decode steps, of fp32 models and of shapes the grouped kernel does not
//     take.  Two launches so that even ONE row spreads over the chip: expert_up_rows (a workgroup = one (row, choice) pair x 8 hidden
//     channels, a wave per channel pair gate / up, lanes across the contraction with 16-byte loads, fp32 sums in a fixed order)
//     leaves the hidden row in the workspace, expert_down_rows (a pair x 16 output channels) consumes it.
//   * grouped matrix-core products for bf16 prompt portions (rows sorted by expert on the device, no host round trip).
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256, NW = NT / 64;
constexpr int FC = 8;             // hidden channels per workgroup of expert_up_rows
constexpr int KC = 16;            // output channels per workgroup of expert_down_rows

// sum_k w[k] * x[k] over this lane's share of n elements; x in LDS (fp32).  VEC: n is a multiple of the 16-byte vector.
template <typename T, bool VEC>
__device__ __forceinline__ float lane_dot(const T* __restrict__ w, const float* __restrict__ x, int n, int lane) {
  float acc = 0.f;
  if constexpr (VEC) {
    constexpr int PER = 16 / sizeof(T);
    for (int k = lane * PER; k < n; k += 64 * PER) {
      const uint4 raw = *reinterpret_cast<const uint4*>(w + k);
      if constexpr (sizeof(T) == 2) {
        const unsigned u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc += __uint_as_float(u[i] << 16) * x[k + 2 * i];
          acc += __uint_as_float(u[i] & 0xFFFF0000u) * x[k + 2 * i + 1];
        }
      } else {
        acc += __uint_as_float(raw.x) * x[k] + __uint_as_float(raw.y) * x[k + 1] + __uint_as_float(raw.z) * x[k + 2] + __uint_as_float(raw.w) * x[k + 3];
      }
    }
  } else {
    for (int k = lane; k < n; k += 64) acc += to_f32(w[k]) * x[k];
  }
  return acc;
}

template <typename T, bool FAST, bool VEC>
__global__ __launch_bounds__(NT) void expert_up_rows(const T* __restrict__ h, const T* __restrict__ gate_up, const int* __restrict__ idx,
                                                    T* __restrict__ act, int K, int F, int top, int kind, float limit) {
  extern __shared__ float hl[];                     // the row [K]
  const int64_t pair = blockIdx.x;
  const int e = idx[pair];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* hr = h + (pair / top) * K;
  for (int k = threadIdx.x; k < K; k += NT) hl[k] = to_f32(hr[k]);
  __syncthreads();
  const T* wg = gate_up + static_cast<int64_t>(e) * 2 * F * K;
  const T* wu = wg + static_cast<int64_t>(F) * K;
  const int f_end = min(F, (static_cast<int>(blockIdx.y) + 1) * FC);
  for (int f = blockIdx.y * FC + wave; f < f_end; f += NW) {
    const float ag = wave_sum(lane_dot<T, VEC>(wg + static_cast<int64_t>(f) * K, hl, K, lane));
    const float au = wave_sum(lane_dot<T, VEC>(wu + static_cast<int64_t>(f) * K, hl, K, lane));
    if (lane == 0) act[pair * F + f] = from_f32<T>(glu_act<FAST>(ag, au, kind, limit, 1.702f));
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(NT) void expert_down_rows(const T* __restrict__ act, const T* __restrict__ down, const int* __restrict__ idx,
                                                      T* __restrict__ y, int K, int F) {
  extern __shared__ float al[];                     // the hidden row [F]
  const int64_t pair = blockIdx.x;
  const int e = idx[pair];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int f = threadIdx.x; f < F; f += NT) al[f] = to_f32(act[pair * F + f]);
  __syncthreads();
  const T* wd = down + static_cast<int64_t>(e) * K * F;
  const int c_end = min(K, (static_cast<int>(blockIdx.y) + 1) * KC);
  for (int c = blockIdx.y * KC + wave; c < c_end; c += NW) {
    const float acc = wave_sum(lane_dot<T, VEC>(wd + static_cast<int64_t>(c) * F, al, F, lane));
    if (lane == 0) y[pair * K + c] = from_f32<T>(acc);
  }
}

template <typename T, bool FAST>
int launch_rows(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t P, int K, int F, int top, int kind, float limit,
                void* ws, hipStream_t s) {
  constexpr int PER = 16 / sizeof(T);
  const bool vec = K % PER == 0 && F % PER == 0 &&
                   (reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(down)) % 16 == 0;
  const dim3 gu(P, (F + FC - 1) / FC), gd(P, (K + KC - 1) / KC);
  const T* hp = static_cast<const T*>(h);
  const T* gp = static_cast<const T*>(gate_up);
  const T* dp = static_cast<const T*>(down);
  T* act = static_cast<T*>(ws);
  if (vec) {
    expert_up_rows<T, FAST, true><<<gu, NT, K * sizeof(float), s>>>(hp, gp, idx, act, K, F, top, kind, limit);
    expert_down_rows<T, true><<<gd, NT, F * sizeof(float), s>>>(act, dp, idx, static_cast<T*>(y), K, F);
  } else {
    expert_up_rows<T, FAST, false><<<gu, NT, K * sizeof(float), s>>>(hp, gp, idx, act, K, F, top, kind, limit);
    expert_down_rows<T, false><<<gd, NT, F * sizeof(float), s>>>(act, dp, idx, static_cast<T*>(y), K, F);
  }
  return after_launch("expert_glu (rows)");
}

}  // namespace

int launch_expert_grouped(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T, int K, int F, int E, int top,
                          int kind, float limit, void* ws, size_t ws_bytes, hipStream_t s);   // mixers_moe_mfma.hip
size_t expert_grouped_workspace(int64_t T, int K, int F, int E, int top);

}  // namespace gbxm

using namespace gbxm;

extern "C" size_t gbxm_expert_glu_workspace(int64_t T_, int32_t K, int32_t F, int32_t E, int32_t top, int32_t act) {
  const size_t rows = static_cast<size_t>(T_) * top * F * (act == GBXM_BF16 ? 2 : 4);      // the hidden rows of the row kernels
  const size_t grouped = act == GBXM_BF16 ? expert_grouped_workspace(T_, K, F, E, top) : 0;
  return grouped > rows ? grouped : rows;
}

extern "C" int gbxm_expert_glu_grouped(int64_t T_, int32_t K, int32_t F, int32_t E, int32_t top, int32_t act) {
  return act == GBXM_BF16 && expert_grouped_workspace(T_, K, F, E, top) > 0;
}

extern "C" int gbxm_expert_glu_act(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T_, int32_t K,
                                   int32_t F, int32_t E, int32_t top, int32_t act, int32_t kind, float limit, void* ws, size_t ws_bytes,
                                   void* stream) {
  if (!h || !gate_up || !down || !idx || !y || K <= 0 || F <= 0 || E <= 0 || top < 1 || top > E || T_ < 0 || (act != GBXM_BF16 && act != GBXM_F32) ||
      (kind != GBXM_GLU_SILU && kind != GBXM_GLU_CLAMPED_SWISH))
    return fail(GBXM_ERR_INVALID, "expert_glu: bad argument");
  if (T_ == 0) return GBXM_OK;
  if (!ws || ws_bytes < gbxm_expert_glu_workspace(T_, K, F, E, top, act)) return fail(GBXM_ERR_INVALID, "expert_glu: workspace too small");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (act == GBXM_BF16) {
    const int rc = launch_expert_grouped(h, gate_up, down, idx, y, T_, K, F, E, top, kind, limit, ws, ws_bytes, s);
    if (rc != GBXM_ERR_UNSUPPORTED) return rc;
  }
  if (static_cast<size_t>(K > F ? K : F) * sizeof(float) > 64 * 1024) return fail(GBXM_ERR_UNSUPPORTED, "expert_glu: rows of %d channels beyond the row kernels' LDS", K > F ? K : F);
  if (T_ * top > 0x7fffffffLL || (F + FC - 1) / FC > 65535 || (K + KC - 1) / KC > 65535) return fail(GBXM_ERR_UNSUPPORTED, "expert_glu: grid");
  return act == GBXM_BF16 ? launch_rows<bf16_t, true>(h, gate_up, down, idx, y, T_ * top, K, F, top, kind, limit, ws, s)
                          : launch_rows<float, false>(h, gate_up, down, idx, y, T_ * top, K, F, top, kind, limit, ws, s);
}

extern "C" int gbxm_expert_glu(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T_, int32_t K, int32_t F,
                               int32_t E, int32_t top, int32_t act, void* ws, size_t ws_bytes, void* stream) {
  return gbxm_expert_glu_act(h, gate_up, down, idx, y, T_, K, F, E, top, act, GBXM_GLU_SILU, 0.f, ws, ws_bytes, stream);
}
