// Recurrent mixers: a decayed matrix state per head.
//
//   recurrent_prep_kernel   short causal convolution + silu on q | k | v, unit q / k heads (a wave per head), q scale, the decay
//                           exp(-rate_h softplus(sign (a + bias))) and beta = sigmoid(b), all in fp32, into one fp32 row.
//   conv_tail_kernel        the last taps-1 convolution inputs of every sequence into its slot.
//   state_scan_kernel<R>    the scan.  The columns of a head's state (one per value channel) never meet: a wave takes four columns, 16
//                           lanes per column, a lane holds R key channels of its column in registers; per token the two dot products
//                           over key channels are R multiply-adds and four cross-lane adds inside a 16-lane row (all 16 lanes end
//                           with the same bits).  Operands come through LDS in chunks of tokens, the next chunk fetched while the
//                           current one is computed.  Sums run in a fixed order: a sequence's result does not depend on what else is
//                           in the step, nor on how many columns a workgroup takes.
//   head_norm_gate_kernel   per-head RMS norm of the read-out, weight and gate, one wave per (row, head).
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256, NW = NT / 64;

// grid (rows, splits): the splits of a row share out its q / k heads (a wave per head, up to MAXD channels a lane in registers),
// its value channels, its decays and betas; a step of few rows takes more splits.  Loads are issued unconditionally (a tap before
// the sequence's start reads a clamped address and counts as zero).
constexpr int MAXD = 4;                     // head channels per lane: heads of up to 256 channels

template <typename T, bool FAST>
__global__ __launch_bounds__(NT) void recurrent_prep_kernel(gbxm_recurrent_prep_args p) {
  const int64_t t = blockIdx.x;
  const int b = p.tok[2 * t], pos = p.tok[2 * t + 1];
  const int slot = p.seq[4 * b], pos0 = p.seq[4 * b + 1], row0 = p.seq[4 * b + 3];
  const int nq = p.G * p.dk, nv = p.H * p.dv, nd = p.H * p.dk;
  const int C = 2 * nq + nv;
  const T* y = static_cast<const T*>(p.y);
  const T* yr = y + t * p.y_stride;
  const T* cw = static_cast<const T*>(p.conv);
  const T* tail = p.taps > 1 ? static_cast<const T*>(p.tail) + static_cast<int64_t>(slot) * (p.taps - 1) * C : nullptr;
  float* out = p.out + t * p.out_stride;
  // channel c of q | k | v after the convolution and silu (or as projected, without a convolution; `plain`: its offset in the row)
  auto value = [&](int c, int plain) {
    if (!cw) { const float x = to_f32(yr[plain]); return p.qkv_silu ? x * sigmoid_<FAST>(x) : x; }
    float acc = 0.f;
    for (int j = 0; j < p.taps; ++j) {
      const int src = pos - (p.taps - 1) + j;
      const bool own = src >= pos0;
      const T* sp = own ? y + (row0 + (src - pos0)) * p.y_stride + p.off_q + c
                        : (tail ? tail + static_cast<int64_t>(max(src, pos0 - (p.taps - 1)) - pos0 + p.taps - 1) * C + c : yr + p.off_q + c);
      const float x = to_f32(*sp);
      acc += src >= 0 ? to_f32(cw[c * p.taps + j]) * x : 0.f;
    }
    return acc * sigmoid_<FAST>(acc);
  };
  const int lane = threadIdx.x & 63;
  const int gwave = blockIdx.y * NW + (threadIdx.x >> 6), n_waves = gridDim.y * NW;
  const int gthread = blockIdx.y * NT + threadIdx.x, n_threads = gridDim.y * NT;
  for (int hd = gwave; hd < 2 * p.G; hd += n_waves) {                  // q heads, then k heads
    const int first = hd * p.dk, plain = (hd < p.G ? p.off_q + first : p.off_k + first - nq);
    float v[MAXD];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAXD; ++i) {
      const int c = lane + 64 * i;
      const bool live = c < p.dk;
      const float x = value(first + (live ? c : 0), plain + (live ? c : 0));
      v[i] = live ? x : 0.f;
      ss += v[i] * v[i];
    }
    float mul = hd < p.G ? p.q_scale : 1.f;
    if (p.unit) mul *= 1.f / sqrtf(wave_sum(ss) + 1e-6f);
#pragma unroll
    for (int i = 0; i < MAXD; ++i)
      if (lane + 64 * i < p.dk) out[first + lane + 64 * i] = v[i] * mul;
  }
  for (int c = gthread; c < nv; c += n_threads) out[2 * nq + c] = value(2 * nq + c, p.off_v + c);
  const T* ar = static_cast<const T*>(p.a) + t * p.a_stride;
  if (!p.a) {                               // no decay projection: the head's constant
    for (int c = gthread; c < nd; c += n_threads) out[2 * nq + nv + c] = p.decay_rate[c / p.dk];
  } else for (int c = gthread; c < nd; c += n_threads) {
    const float z = p.sign * (to_f32(ar[c]) + p.decay_bias[c]);
    const float sp = z > 20.f ? z : log1p_<FAST>(exp_<FAST>(z));
    out[2 * nq + nv + c] = exp_<FAST>(-p.decay_rate[c / p.dk] * sp);
  }
  if (p.off_beta >= 0)
    for (int c = gthread; c < p.H; c += n_threads) out[2 * nq + nv + nd + c] = sigmoid_<FAST>(to_f32(yr[p.off_beta + c]));
}

template <typename T>
__global__ __launch_bounds__(NT) void conv_tail_kernel(const T* __restrict__ y, int64_t y_stride, T* __restrict__ tail, const int* __restrict__ seq,
                                                      int C, int taps) {
  const int b = blockIdx.y;
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], n = seq[4 * b + 2], row0 = seq[4 * b + 3];
  const int keep = taps - 1;
  T* tl = tail + static_cast<int64_t>(slot) * keep * C;
  for (int c = blockIdx.x * NT + threadIdx.x; c < C; c += gridDim.x * NT) {
    // entry i afterwards holds position pos0 + n - keep + i: ascending i reads entries above the ones already written
    for (int i = 0; i < keep; ++i) {
      const int pos = pos0 + n - keep + i;
      T v;
      if (pos >= pos0) v = y[(row0 + (pos - pos0)) * y_stride + c];
      else if (pos >= 0) v = tl[static_cast<int64_t>(i + n) * C + c];
      else v = from_f32<T>(0.f);
      tl[static_cast<int64_t>(i) * C + c] = v;
    }
  }
}

// Sum over the 16 lanes of a row; every lane of the row gets the same bits (each step adds the two halves of a mirrored pair).
__device__ __forceinline__ float row16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false));    // quad_perm [1,0,3,2]
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false));    // quad_perm [2,3,0,1]
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false));   // row_half_mirror
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, false));   // row_mirror
  return v;
}

// NW waves per workgroup = 4 NW columns of one (sequence, head).  The operands of CH tokens (q | k | decay padded to 16 R channels, the
// workgroup's value columns, beta) are staged in LDS, shared by the waves, two buffers: the next chunk is fetched into registers before
// the current one is computed and parked in the other buffer afterwards, one barrier per chunk.  Lane ks of a 16-lane row owns the key
// channels ks, ks + 16, ...: LDS reads and the state's loads and stores are contiguous over the row.
template <int R, bool DELTA, int NW>
__global__ __launch_bounds__(64 * NW) void state_scan_kernel(const float* __restrict__ r, int64_t r_stride, float* __restrict__ state,
                                                            float* __restrict__ out, const int* __restrict__ seq, int H, int G, int dk, int dv) {
  constexpr int DKP = 16 * R, NCOL = 4 * NW, ROW = 3 * DKP + NCOL + 1, NTH = 64 * NW;
  constexpr int CH = NW == 1 ? (R <= 4 ? 4 : 2) : (R <= 4 ? 32 : (R <= 8 ? 16 : 8)) * NW / 4;     // one-wave workgroups serve steps of few rows
  constexpr int PF = (CH * ROW + NTH - 1) / NTH;
  __shared__ float buf[2][CH * ROW];
  const int b = blockIdx.z, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, ks = lane & 15;
  const int col0 = blockIdx.x * NCOL, lcol = wave * 4 + (lane >> 4), col = col0 + lcol;
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], n = seq[4 * b + 2], row0 = seq[4 * b + 3];
  const bool col_ok = col < dv;
  const int colc = col_ok ? col : dv - 1;
  const int nq = G * dk, nv = H * dv;
  const int g = h / (H / G);
  float* sp = state + ((static_cast<int64_t>(slot) * H + h) * dv + colc) * dk + min(ks, dk - 1);     // (a lane past the last channel holds zeros)
  // every load below is issued unconditionally from an address inside the buffers (what it must not deliver is replaced afterwards):
  // loads under a branch wait for one another, and a chunk's fetch then costs the sum of their latencies
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = sp[ks + 16 * i < dk ? 16 * i : 0];
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = (pos0 > 0 && ks + 16 * i < dk) ? S[i] : 0.f;
  const float* base = r + static_cast<int64_t>(row0) * r_stride;
  const int oq = g * dk, ok = nq + g * dk, ov = 2 * nq + h * dv, og = 2 * nq + nv + h * dk, ob = 2 * nq + nv + H * dk + h;
  float pf[PF];
  int offs[PF], tts[PF];                    // where slot i of this thread's share of a chunk comes from: token of the chunk, offset in its row
  unsigned loaded = 0;                      // bit i: pf[i] is an operand (else the slot's neutral value: 1 for a decay, 0 elsewhere)
#pragma unroll
  for (int i = 0; i < PF; ++i) {
    const int idx = min(static_cast<int>(threadIdx.x) + i * NTH, CH * ROW - 1);
    const int tt = idx / ROW, j = idx - tt * ROW;
    const int seg = j < DKP ? 0 : (j < 2 * DKP ? 1 : (j < 3 * DKP ? 2 : 3));
    const int jj = j - seg * DKP;                                     // segment 3: the value columns, then beta
    const bool is_beta = seg == 3 && jj == NCOL;
    const int first = seg == 0 ? oq : (seg == 1 ? ok : (seg == 2 ? og : ov + col0));
    const int count = seg < 3 ? dk : min(dv - col0, NCOL);
    const bool valid = is_beta ? DELTA : jj < count;
    offs[i] = valid ? (is_beta ? ob : first + jj) : oq;
    tts[i] = tt;
    loaded |= static_cast<unsigned>(valid) << i;
  }
  auto fetch = [&](int t0) {
    const float* cb = base + static_cast<int64_t>(t0) * r_stride;
    if (t0 + CH <= n) {
#pragma unroll
      for (int i = 0; i < PF; ++i) pf[i] = cb[static_cast<int64_t>(tts[i]) * r_stride + offs[i]];
    } else {                                // the sequence's last chunk: rows past its end are read as its last row (and never used)
      const int last = n - 1 - t0;
#pragma unroll
      for (int i = 0; i < PF; ++i) pf[i] = cb[static_cast<int64_t>(min(tts[i], last)) * r_stride + offs[i]];
    }
  };
  auto park = [&](float* dst) {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int idx = threadIdx.x + i * NTH;
      const int j = idx % ROW;
      const float neutral = ((j >= 2 * DKP && j < 3 * DKP) || j == ROW - 1) ? 1.f : 0.f;
      if (idx < CH * ROW) dst[idx] = ((loaded >> i) & 1u) ? pf[i] : neutral;
    }
  };
  fetch(0);
  park(buf[0]);
  __syncthreads();
  float* op = out + static_cast<int64_t>(row0) * nv + h * dv + colc;
  int which = 0;
  for (int t0 = 0; t0 < n; t0 += CH, which ^= 1) {
    const bool more = t0 + CH < n;
    if (more) fetch(t0 + CH);
    const float* cur = buf[which];
    const int cn = min(CH, n - t0);
#pragma unroll 2
    for (int tt = 0; tt < cn; ++tt) {
      const float* row = cur + tt * ROW;
      float q[R], k[R];
#pragma unroll
      for (int i = 0; i < R; ++i) {
        q[i] = row[ks + 16 * i];
        k[i] = row[DKP + ks + 16 * i];
        S[i] *= row[2 * DKP + ks + 16 * i];
      }
      float u = row[3 * DKP + lcol];
      if constexpr (DELTA) {
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) dot += k[i] * S[i];
        u = row[3 * DKP + NCOL] * (u - row16_sum(dot));
      }
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) { S[i] += k[i] * u; o += q[i] * S[i]; }
      o = row16_sum(o);
      if (ks == 0 && col_ok) op[static_cast<int64_t>(t0 + tt) * nv] = o;
    }
    if (more) park(buf[which ^ 1]);
    __syncthreads();
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (ks + 16 * i < dk) sp[16 * i] = S[i];
  }
}

template <typename T, bool FAST>
__global__ __launch_bounds__(NT) void head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate, int64_t gate_stride,
                                                           const float* __restrict__ w, T* __restrict__ out, int H, int dv, float eps, int kind) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int h = blockIdx.y * NW + (threadIdx.x >> 6);
  if (h >= H) return;
  const float* x = o + (t * H + h) * dv;
  float ss = 0.f;
  for (int c = lane; c < dv; c += 64) ss += x[c] * x[c];
  const float r = 1.f / sqrtf(wave_sum(ss) / dv + eps);
  const T* g = gate + t * gate_stride + h * dv;
  T* y = out + (t * H + h) * dv;
  for (int c = lane; c < dv; c += 64) {
    const float z = to_f32(g[c]);
    const float s = sigmoid_<FAST>(z);
    y[c] = from_f32<T>(x[c] * r * w[c] * (kind == 1 ? z * s : s));
  }
}

template <bool DELTA, int NW>
int launch_scan(int R, int B, hipStream_t s, const float* r, int64_t r_stride, float* state, float* out, const int32_t* seq, int H, int G, int dk,
                int dv) {
  const dim3 grid((dv + 4 * NW - 1) / (4 * NW), H, B);
#define GBXM_SCAN(N) state_scan_kernel<N, DELTA, NW><<<grid, 64 * NW, 0, s>>>(r, r_stride, state, out, seq, H, G, dk, dv)
  if (R <= 1) GBXM_SCAN(1);
  else if (R <= 2) GBXM_SCAN(2);
  else if (R <= 3) GBXM_SCAN(3);
  else if (R <= 4) GBXM_SCAN(4);
  else if (R <= 6) GBXM_SCAN(6);
  else if (R <= 8) GBXM_SCAN(8);
  else if (R <= 12) GBXM_SCAN(12);
  else GBXM_SCAN(16);
#undef GBXM_SCAN
  return after_launch("state_scan");
}

bool act_ok(int act) { return act == GBXM_BF16 || act == GBXM_F32; }

}  // namespace
}  // namespace gbxm

using namespace gbxm;

extern "C" {

int gbxm_recurrent_prepare(const gbxm_recurrent_prep_args* a, void* stream) {
  if (!a || !act_ok(a->act) || !a->y || (a->a && !a->decay_bias) || !a->decay_rate || !a->seq || !a->tok || !a->out || a->T < 0 || a->H < 1 || a->G < 1 ||
      a->H % a->G || a->dk < 1 || a->dv < 1 || a->off_q < 0 || a->off_k < 0 || a->off_v < 0)
    return fail(GBXM_ERR_INVALID, "recurrent_prepare: bad argument");
  const int nq = a->G * a->dk, nv = a->H * a->dv, C = 2 * nq + nv;
  if (a->conv && (a->taps < 1 || (a->taps > 1 && !a->tail) || a->off_k != a->off_q + nq || a->off_v != a->off_k + nq))
    return fail(GBXM_ERR_INVALID, "recurrent_prepare: a convolution needs q | k | v side by side and the slots' tails");
  if (a->out_stride < C + a->H * a->dk + (a->off_beta >= 0 ? a->H : 0)) return fail(GBXM_ERR_INVALID, "recurrent_prepare: output rows too short");
  if (a->dk > 64 * MAXD) return fail(GBXM_ERR_UNSUPPORTED, "recurrent_prepare: heads of %d channels (at most %d)", a->dk, 64 * MAXD);
  if (a->T == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // splits of a row: enough workgroups for the chip when the step has few rows, never more than the row has work for
  int64_t splits = (1024 + a->T - 1) / a->T;
  const int64_t most = (C + a->H * a->dk + 4 * NT - 1) / (4 * NT);
  if (splits > most) splits = most;
  if (splits > 64) splits = 64;
  if (splits < 1) splits = 1;
  const dim3 grid(a->T, static_cast<unsigned>(splits));
  if (a->act == GBXM_BF16) recurrent_prep_kernel<bf16_t, false><<<grid, NT, 0, s>>>(*a);
  else recurrent_prep_kernel<float, false><<<grid, NT, 0, s>>>(*a);
  return after_launch("recurrent_prepare");
}

int gbxm_conv_tail_update(const void* y, int64_t y_stride, void* tail, const int32_t* seq, int32_t B, int32_t C, int32_t taps, int32_t act,
                          void* stream) {
  if (!act_ok(act) || !y || !tail || !seq || B < 0 || C < 1 || taps < 2 || y_stride < C) return fail(GBXM_ERR_INVALID, "conv_tail_update: bad argument");
  if (B == 0) return GBXM_OK;
  if (B > 65535) return fail(GBXM_ERR_UNSUPPORTED, "conv_tail_update: more than 65535 sequences in a step");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((C + NT - 1) / NT, B);
  if (act == GBXM_BF16) conv_tail_kernel<bf16_t><<<grid, NT, 0, s>>>(static_cast<const bf16_t*>(y), y_stride, static_cast<bf16_t*>(tail), seq, C, taps);
  else conv_tail_kernel<float><<<grid, NT, 0, s>>>(static_cast<const float*>(y), y_stride, static_cast<float*>(tail), seq, C, taps);
  return after_launch("conv_tail_update");
}

int gbxm_state_scan(const float* r, int64_t r_stride, float* state, float* out, const int32_t* seq, int32_t B, int64_t T_, int32_t H, int32_t G,
                    int32_t dk, int32_t dv, int32_t delta, void* stream) {
  if (!r || !state || !out || !seq || B < 0 || H < 1 || G < 1 || H % G || dk < 1 || dv < 1 ||
      r_stride < 2 * G * dk + H * dv + H * dk + (delta ? H : 0))
    return fail(GBXM_ERR_INVALID, "state_scan: bad argument");
  if (dk > 256) return fail(GBXM_ERR_UNSUPPORTED, "state_scan: %d key channels per head (at most 256)", dk);
  if (B == 0) return GBXM_OK;
  if (B > 65535 || H > 65535) return fail(GBXM_ERR_UNSUPPORTED, "state_scan: grid");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int R = (dk + 15) / 16;
  // long rows (prompts): 16 columns per workgroup share the staged operands; a few rows per sequence: 4 columns, four times the
  // workgroups for the state's traffic.  A column's arithmetic is the same in both.
  if (T_ >= 8 * static_cast<int64_t>(B))
    return delta ? launch_scan<true, 4>(R, B, s, r, r_stride, state, out, seq, H, G, dk, dv)
                 : launch_scan<false, 4>(R, B, s, r, r_stride, state, out, seq, H, G, dk, dv);
  return delta ? launch_scan<true, 1>(R, B, s, r, r_stride, state, out, seq, H, G, dk, dv)
               : launch_scan<false, 1>(R, B, s, r, r_stride, state, out, seq, H, G, dk, dv);
}

int gbxm_head_norm_gate(const float* o, const void* gate, int64_t gate_stride, const float* w, void* out, int64_t T_, int32_t H, int32_t dv,
                        float eps, int32_t kind, int32_t act, void* stream) {
  if (!act_ok(act) || !o || !gate || !w || !out || T_ < 0 || H < 1 || dv < 1 || gate_stride < H * dv || (kind != 1 && kind != 2))
    return fail(GBXM_ERR_INVALID, "head_norm_gate: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(T_, (H + NW - 1) / NW);
  if (act == GBXM_BF16)
    head_norm_gate_kernel<bf16_t, false><<<grid, NT, 0, s>>>(o, static_cast<const bf16_t*>(gate), gate_stride, w, static_cast<bf16_t*>(out), H, dv, eps, kind);
  else
    head_norm_gate_kernel<float, false><<<grid, NT, 0, s>>>(o, static_cast<const float*>(gate), gate_stride, w, static_cast<float*>(out), H, dv, eps, kind);
  return after_launch("head_norm_gate");
}

}  // extern "C"
