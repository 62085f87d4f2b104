// Softmax attention with a sink over a ragged step, and the row kernels around it: head rotations / norms, the append to slot
// tables, the parallel-layer stream update and the feed-forward activation.
//
//   out[t][h] = gate[t][h] * sum_j p_j v_j,   p_j = exp(s_j) / (exp(sink_h) + sum_j exp(s_j)),   s_j = scale <q[t][h], k_j>
// over the keys j <= i of the row's sequence with i - j < window or j < keep.  The keys a row sees are two runs of positions,
// [0, min(keep, lo)) and [lo, i] with lo = max(0, i - window + 1); the kernels walk them as ONE run of indices (no masked key is
// ever loaded).  Position j of a sequence is read from its slot's table (row j if j < keep, else keep + (j - keep) % ring) when it
// lies before the step, and from the step's own rows otherwise.
//
// sink_rows_kernel: any head sizes, fp32 or bf16, all arithmetic fp32 -- one workgroup per (row, kv head, chunk of its query
// heads, share of the key tiles); scores by a thread per (head, key) of a 64-key tile, running maximum / sum per head in LDS, the
// value sum with a wave per key and the lanes across channels.  A step of few rows splits the key tiles over workgroups; each
// leaves (sum, maximum, denominator) and sink_reduce_kernel joins them in a fixed order, adds the sink and applies the gate.
// The matrix-core kernel for bf16 prompt portions is in mixers_sink_mfma.hip.
#include <algorithm>
#include <climits>
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256, NW = NT / 64;
constexpr int KT = 64;            // keys per tile
constexpr int RC = 8;             // query heads a workgroup takes at most
constexpr int DCH = 128;          // value channels per lane pass (two per lane)
constexpr int NCH = 4;            // lane passes: value sizes up to NCH * DCH

struct SinkGeo {
  int H, G, dk, dv, window, keep, ring;
  float scale;
  int64_t q_row, q_head, k_row, k_head, v_row, v_head, kc_slot, kc_row, kc_head, vc_slot, vc_row, vc_head, gate_row;
};

template <typename T, bool VEC>
__device__ __forceinline__ float dot_row(const float* __restrict__ q, const T* __restrict__ k, int dk) {
  float dot = 0.f;
  if constexpr (VEC) {
    constexpr int PER = 16 / sizeof(T);
    for (int d = 0; d < dk; d += PER) {
      const uint4 raw = *reinterpret_cast<const uint4*>(k + d);
      if constexpr (sizeof(T) == 2) {
        const unsigned u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          dot += q[d + 2 * i] * __uint_as_float(u[i] << 16);
          dot += q[d + 2 * i + 1] * __uint_as_float(u[i] & 0xFFFF0000u);
        }
      } else {
        dot += q[d] * __uint_as_float(raw.x) + q[d + 1] * __uint_as_float(raw.y) + q[d + 2] * __uint_as_float(raw.z) + q[d + 3] * __uint_as_float(raw.w);
      }
    }
  } else {
    for (int d = 0; d < dk; ++d) dot += q[d] * to_f32(k[d]);
  }
  return dot;
}

template <typename T, bool FAST, bool VEC>
__global__ __launch_bounds__(NT) void sink_rows_kernel(const T* __restrict__ q, const T* __restrict__ kn, const T* __restrict__ vn,
                                                      const T* __restrict__ kc, const T* __restrict__ vc, const int* __restrict__ seq,
                                                      const int* __restrict__ tok, T* __restrict__ out, const float* __restrict__ sink,
                                                      const T* __restrict__ gate, SinkGeo g, int rc, int splits, float* __restrict__ partial) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const T** kptr = reinterpret_cast<const T**>(lds_raw);            // [KT] rows of the tile's keys
  const T** vptr = kptr + KT;                                        // [KT] and values
  float* ql = reinterpret_cast<float*>(vptr + KT);                   // [rc][dk]
  float* gl = ql + rc * g.dk;                                        // [rc][KT] scores, then weights
  float* ml = gl + rc * KT;                                          // [rc] running maximum
  float* ll = ml + rc;                                               // [rc] running denominator
  float* al = ll + rc;                                               // [rc] rescale of this tile
  float* sums = al + rc;                                             // [NW][rc * dv]
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int R = g.H / g.G;
  const int chunks = (R + rc - 1) / rc;
  const int kvh = blockIdx.y / chunks, r0 = (blockIdx.y % chunks) * rc;
  const int nr = min(rc, R - r0);                   // query heads of this workgroup: kvh * R + r0 + (0 .. nr-1)
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], row0 = seq[4 * b + 3];
  const int head0 = kvh * R + r0;
  for (int i = threadIdx.x; i < nr * g.dk; i += NT) ql[i] = to_f32(q[t * g.q_row + (head0 + i / g.dk) * g.q_head + i % g.dk]);
  if (threadIdx.x < nr) {
    const bool own_sink = sink && splits == 1;      // split key tiles: the sink joins in the reduce
    ml[threadIdx.x] = own_sink ? sink[head0 + threadIdx.x] : -INFINITY;
    ll[threadIdx.x] = own_sink ? 1.f : 0.f;
  }
  float acc[NCH][RC][2];
#pragma unroll
  for (int c = 0; c < NCH; ++c)
#pragma unroll
    for (int r = 0; r < RC; ++r) acc[c][r][0] = acc[c][r][1] = 0.f;
  const bool pair_loads = g.dv % 2 == 0 && VEC;
  // the visible keys as one run of indices: [0, na) are positions 0 .. na-1 (kept first tokens that left the window), the rest lo ..
  const int lo = g.window > 0 ? max(0, pos - g.window + 1) : 0;
  const int na = min(g.keep, lo);
  const int total = na + (pos - lo + 1);
  for (int it = static_cast<int>(blockIdx.z) * KT; it < total; it += KT * splits) {
    __syncthreads();                                // the previous tile's weights and rows have been consumed
    if (threadIdx.x < KT) {
      const int iv = min(it + static_cast<int>(threadIdx.x), total - 1);
      const int j = iv < na ? iv : lo + (iv - na);
      if (j < pos0) {
        const int64_t row = j < g.keep ? j : g.keep + (j - g.keep) % g.ring;
        kptr[threadIdx.x] = kc + slot * g.kc_slot + row * g.kc_row + kvh * g.kc_head;
        vptr[threadIdx.x] = vc + slot * g.vc_slot + row * g.vc_row + kvh * g.vc_head;
      } else {
        const int64_t row = row0 + (j - pos0);
        kptr[threadIdx.x] = kn + row * g.k_row + kvh * g.k_head;
        vptr[threadIdx.x] = vn + row * g.v_row + kvh * g.v_head;
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nr * KT; i += NT) {
      const int r = i / KT, jj = i % KT;
      gl[i] = it + jj < total ? dot_row<T, VEC>(ql + r * g.dk, kptr[jj], g.dk) * g.scale : -INFINITY;
    }
    __syncthreads();
    for (int r = wave; r < nr; r += NW) {           // a wave per head: the tile's maximum, the weights, their sum
      const float s = gl[r * KT + lane];
      float mx = s;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      const float m_old = ml[r], m_new = fmaxf(m_old, mx);            // mx is finite: a tile holds at least one key
      const float p = exp_<FAST>(s - m_new);
      gl[r * KT + lane] = p;
      const float ps = wave_sum(p);
      if (lane == 0) {
        const float alpha = exp_<FAST>(m_old - m_new);                // exp(-inf) = 0 at the first tile without a sink
        ml[r] = m_new; ll[r] = ll[r] * alpha + ps; al[r] = alpha;
      }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < RC; ++r)
      if (r < nr) {
        const float alpha = al[r];
#pragma unroll
        for (int c = 0; c < NCH; ++c) { acc[c][r][0] *= alpha; acc[c][r][1] *= alpha; }
      }
    const int nj = min(KT, total - it);
#pragma unroll 4
    for (int jj = wave; jj < nj; jj += NW) {
      const T* vr = vptr[jj];
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const int d0 = c * DCH + 2 * lane;
        if (d0 < g.dv) {
          float v0, v1 = 0.f;
          if (pair_loads) {
            if constexpr (sizeof(T) == 2) {
              const unsigned u = *reinterpret_cast<const unsigned*>(vr + d0);
              v0 = __uint_as_float(u << 16); v1 = __uint_as_float(u & 0xFFFF0000u);
            } else {
              const float2 f = *reinterpret_cast<const float2*>(vr + d0);
              v0 = f.x; v1 = f.y;
            }
          } else {
            v0 = to_f32(vr[d0]);
            if (d0 + 1 < g.dv) v1 = to_f32(vr[d0 + 1]);
          }
#pragma unroll
          for (int r = 0; r < RC; ++r)
            if (r < nr) {
              const float p = gl[r * KT + jj];
              acc[c][r][0] += p * v0;
              acc[c][r][1] += p * v1;
            }
        }
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int d0 = c * DCH + 2 * lane;
    if (d0 < g.dv)
#pragma unroll
      for (int r = 0; r < RC; ++r)
        if (r < nr) {
          sums[(wave * rc + r) * g.dv + d0] = acc[c][r][0];
          if (d0 + 1 < g.dv) sums[(wave * rc + r) * g.dv + d0 + 1] = acc[c][r][1];
        }
  }
  __syncthreads();
  if (splits > 1) {
    const int pw = partial_width(g.dv);
    float* prow = partial + ((static_cast<int64_t>(blockIdx.z) * gridDim.x + t) * g.H + head0) * pw;
    for (int i = threadIdx.x; i < nr * g.dv; i += NT) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) s += sums[w * rc * g.dv + i];
      prow[(i / g.dv) * pw + i % g.dv] = s;
    }
    if (threadIdx.x < nr) {
      prow[threadIdx.x * pw + pw - 2] = ml[threadIdx.x];
      prow[threadIdx.x * pw + pw - 1] = ll[threadIdx.x];
    }
    return;
  }
  T* orow = out + t * (static_cast<int64_t>(g.H) * g.dv) + head0 * g.dv;
  for (int i = threadIdx.x; i < nr * g.dv; i += NT) {
    const int r = i / g.dv;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) s += sums[w * rc * g.dv + i];
    s /= ll[r];
    if (gate) s *= sigmoid_<FAST>(to_f32(gate[t * g.gate_row + head0 + r]));
    orow[i] = from_f32<T>(s);
  }
}

// One workgroup per (row, head): joins the key splits' (sum, maximum, denominator) in split order, adds the sink, applies the gate.
// Rows of `partial` are partial_width(dv) floats (the sums, padding to a multiple of four, maximum, denominator), so a thread
// reads four channels at once; the two halves of the workgroup take the even and the odd splits and meet in LDS.
template <typename T, bool FAST>
__global__ __launch_bounds__(256) void sink_reduce_kernel(const float* __restrict__ partial, T* __restrict__ out, const float* __restrict__ sink,
                                                         const T* __restrict__ gate, int64_t gate_row, int64_t T_, int H, int dv, int splits) {
  __shared__ float wz[64];
  __shared__ float den;
  __shared__ float4 other[128];
  const int64_t t = blockIdx.x;
  const int head = blockIdx.y, pw = partial_width(dv);
  const int64_t zs = T_ * H * pw;
  const float* p0 = partial + (t * H + head) * pw;
  if (threadIdx.x < 64) {
    const int z = threadIdx.x;
    const float m = z < splits ? p0[z * zs + pw - 2] : -INFINITY;
    float top = m;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) top = fmaxf(top, __shfl_xor(top, o, 64));
    if (sink) top = fmaxf(top, sink[head]);
    const float w = z < splits ? exp_<FAST>(m - top) : 0.f;
    wz[z] = w;
    float l = z < splits ? w * p0[z * zs + pw - 1] : 0.f;
    l = wave_sum(l);
    if (z == 0) den = l + (sink ? exp_<FAST>(sink[head] - top) : 0.f);
  }
  __syncthreads();
  const float f = (gate ? sigmoid_<FAST>(to_f32(gate[t * gate_row + head])) : 1.f) / den;
  const int half = threadIdx.x >> 7, q = threadIdx.x & 127;
  for (int d0 = 0; d0 < dv; d0 += 512) {
    const int d = d0 + 4 * q;
    float4 s = float4{0.f, 0.f, 0.f, 0.f};
    if (d < dv)
#pragma unroll 4
      for (int z = half; z < splits; z += 2) {
        const float4 v = *reinterpret_cast<const float4*>(p0 + z * zs + d);      // (channels past dv inside the last four are padding)
        const float w = wz[z];
        s.x += w * v.x; s.y += w * v.y; s.z += w * v.z; s.w += w * v.w;
      }
    __syncthreads();
    if (half) other[q] = s;
    __syncthreads();
    if (!half && d < dv) {
      const float4 u = other[q];
      const float r[4] = {(s.x + u.x) * f, (s.y + u.y) * f, (s.z + u.z) * f, (s.w + u.w) * f};
      for (int c = 0; c < 4 && d + c < dv; ++c) out[(t * H + head) * dv + d + c] = from_f32<T>(r[c]);
    }
  }
}

template <typename T, bool FAST>
int launch_rows(const gbxm_sink_attn_args& a, const SinkGeo& g, int rc, int chunks, size_t lds, hipStream_t s) {
  constexpr int PER = 16 / sizeof(T);
  auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  bool vec = a.dk % PER == 0 && a.k_row % PER == 0 && a.k_head % PER == 0 && al(a.k_new) && a.v_row % 2 == 0 && a.v_head % 2 == 0 &&
             reinterpret_cast<uintptr_t>(a.v_new) % 8 == 0;
  if (a.kcache)
    vec = vec && a.kc_slot % PER == 0 && a.kc_row % PER == 0 && a.kc_head % PER == 0 && al(a.kcache) && a.vc_slot % 2 == 0 && a.vc_row % 2 == 0 &&
          a.vc_head % 2 == 0 && reinterpret_cast<uintptr_t>(a.vcache) % 8 == 0;
  int splits = 1;
  const int64_t groups = a.T * a.G * chunks;
  if (a.partial && a.partial_splits > 1 && groups < 256) {
    splits = static_cast<int>(std::min<int64_t>(std::min<int64_t>(512 / groups, 64), a.partial_splits));
    if (splits < 2) splits = 1;
  }
  const dim3 grid(a.T, a.G * chunks, splits);
  const T* q = static_cast<const T*>(a.q);
  const T* kn = static_cast<const T*>(a.k_new);
  const T* vn = static_cast<const T*>(a.v_new);
  const T* kc = static_cast<const T*>(a.kcache);
  const T* vc = static_cast<const T*>(a.vcache);
  const T* gate = static_cast<const T*>(a.gate);
  T* out = static_cast<T*>(a.out);
  float* part = static_cast<float*>(a.partial);
  if (vec)
    sink_rows_kernel<T, FAST, true><<<grid, NT, lds, s>>>(q, kn, vn, kc, vc, a.seq, a.tok, out, a.sink, gate, g, rc, splits, part);
  else
    sink_rows_kernel<T, FAST, false><<<grid, NT, lds, s>>>(q, kn, vn, kc, vc, a.seq, a.tok, out, a.sink, gate, g, rc, splits, part);
  if (splits > 1) sink_reduce_kernel<T, FAST><<<dim3(a.T, a.H), 256, 0, s>>>(part, out, a.sink, gate, a.gate_row, a.T, a.H, a.dv, splits);
  return after_launch("sink_attention (rows)");
}

// ------------------------------------------------------------------------------------------------ rotations and norms of heads
struct Segments {
  gbxm_head_segment s[GBXM_MAX_SEGMENTS];
};

// One workgroup per (row, segment); its waves take the segment's heads four at a time.  A head is staged in LDS as fp32, every
// lane forms its rotated channels from there (its own and the partner of the pair), the statistic is a wave sum.
template <typename T>
__global__ __launch_bounds__(NT) void rotate_norm_kernel(T* __restrict__ rows, int64_t stride, const int* __restrict__ positions, int64_t pos_stride,
                                                        Segments segs, float eps, int max_dim) {
  extern __shared__ float head_lds[];               // [NW][2][max_dim], then cos [max_dim / 2], sin [max_dim / 2]
  const gbxm_head_segment sg = segs.s[blockIdx.y];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* in = head_lds + wave * 2 * max_dim;
  float* turned = in + max_dim;
  float* cs_t = head_lds + NW * 2 * max_dim;
  float* sn_t = cs_t + max_dim / 2 + 1;
  const float pos = static_cast<float>(positions[blockIdx.x * pos_stride]);
  const int half = sg.rot_dims / 2;
  for (int i = threadIdx.x; i < half; i += NT) {    // the row's angles once, for all heads of the segment
    float sn, cs;
    sincosf(pos * sg.freq[i], &sn, &cs);
    cs_t[i] = cs * sg.mult;
    sn_t[i] = sn * sg.mult * sg.sign;
  }
  for (int h0 = 0; h0 < sg.heads; h0 += NW) {
    const int head = h0 + wave;
    const bool live = head < sg.heads;
    T* p = rows + blockIdx.x * stride + sg.offset + static_cast<int64_t>(live ? head : 0) * sg.head_dim;
    __syncthreads();
    if (live)
      for (int c = lane; c < sg.head_dim; c += 64) in[c] = to_f32(p[c]);
    __syncthreads();
    if (sg.norm >= 3) {                             // norm before the rotation: the staged head is replaced by its normed image
      if (live) {
        float s0 = 0.f;
        for (int c = lane; c < sg.head_dim; c += 64) s0 += in[c] * in[c];
        const float r0 = 1.f / sqrtf(wave_sum(s0) / sg.head_dim + eps);
        for (int c = lane; c < sg.head_dim; c += 64) in[c] = in[c] * r0 * (sg.norm == 4 ? sg.weight[c] : 1.f);
      }
      __syncthreads();
    }
    if (!live) continue;
    float ss = 0.f;
    for (int c = lane; c < sg.head_dim; c += 64) {
      float v = in[c];
      const int idx = c - sg.rot_offset;
      if (idx >= 0 && idx < sg.rot_dims) {
        int i, other;
        bool first;
        if (sg.interleaved) { i = idx >> 1; first = !(idx & 1); other = first ? c + 1 : c - 1; }
        else { first = idx < half; i = first ? idx : idx - half; other = first ? c + half : c - half; }
        const float sn = sn_t[i], cs = cs_t[i];
        // (u, w) -> (u cos - w sin, w cos + u sin)
        v = first ? v * cs - in[other] * sn : v * cs + in[other] * sn;
      }
      turned[c] = v;
      ss += v * v;
    }
    float r = 1.f;
    if (sg.norm == 1 || sg.norm == 2) r = 1.f / sqrtf(wave_sum(ss) / sg.head_dim + eps);
    for (int c = lane; c < sg.head_dim; c += 64) {
      float v = turned[c] * r;
      if (sg.norm == 2) v *= sg.weight[c];
      p[c] = from_f32<T>(v);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void stream_add_kernel(float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x;
  if (i >= n) return;
  float y = to_f32(a[i]);
  if (b) y += to_f32(b[i]);
  x[i] += y;
}

// x += a (+ b), then h = rms_norm(x) * w in the activation dtype: a parallel layer's stream update and the next layer's norm.
template <typename T>
__global__ __launch_bounds__(NT) void stream_add_norm_kernel(float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b,
                                                            const float* __restrict__ w, T* __restrict__ h, int width, float eps) {
  __shared__ float red[NW];
  const int64_t t = blockIdx.x;
  float* xr = x + t * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += NT) {
    float y = to_f32(a[t * width + c]);
    if (b) y += to_f32(b[t * width + c]);
    const float v = xr[c] + y;
    xr[c] = v;
    ss += v * v;
  }
  ss = block_sum<NW>(ss, red);
  const float r = 1.f / sqrtf(ss / width + eps);
  for (int c = threadIdx.x; c < width; c += NT) h[t * width + c] = from_f32<T>(xr[c] * r * w[c]);      // (each thread re-reads what it wrote)
}

// out[t][h][j] = sum_i in[t][h][i] w[h][i][j] for j < n_out, then out[t][h][n_out + c] = in[t][h][n_in + c] for c < n_tail: a small
// matrix of its own per head, applied to few rows (single-row steps): one workgroup per (row, head), the head's input in LDS,
// threads across the outputs (coalesced reads of w), fp32 sums.
template <typename T>
__global__ __launch_bounds__(NT) void head_project_kernel(const T* __restrict__ in, int64_t in_row, int64_t in_head, const T* __restrict__ w,
                                                         T* __restrict__ out, int64_t out_row, int64_t out_head, int n_in, int n_out, int n_tail) {
  extern __shared__ float xin[];                   // [n_in]
  const T* ip = in + blockIdx.x * in_row + blockIdx.y * in_head;
  T* op = out + blockIdx.x * out_row + blockIdx.y * out_head;
  const T* wp = w + static_cast<int64_t>(blockIdx.y) * n_in * n_out;
  for (int i = threadIdx.x; i < n_in; i += NT) xin[i] = to_f32(ip[i]);
  __syncthreads();
  for (int j = threadIdx.x; j < n_out; j += NT) {
    float s4[4] = {0.f, 0.f, 0.f, 0.f};
    int i = 0;
    for (; i + 4 <= n_in; i += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) s4[u] += xin[i + u] * to_f32(wp[static_cast<int64_t>(i + u) * n_out + j]);
    }
    for (; i < n_in; ++i) s4[i & 3] += xin[i] * to_f32(wp[static_cast<int64_t>(i) * n_out + j]);
    op[j] = from_f32<T>((s4[0] + s4[1]) + (s4[2] + s4[3]));
  }
  for (int c = threadIdx.x; c < n_tail; c += NT) op[n_out + c] = ip[n_in + c];
}

// The same with 16-byte loads of w: a thread owns a run of PER outputs and every IS-th input channel (IS = 256 / (outputs / PER):
// all threads stream w, many loads in flight each); the IS partial sums of an output meet in LDS in a fixed order.
template <typename T>
__global__ __launch_bounds__(NT) void head_project_vec_kernel(const T* __restrict__ in, int64_t in_row, int64_t in_head, const T* __restrict__ w,
                                                             T* __restrict__ out, int64_t out_row, int64_t out_head, int n_in, int n_out, int n_tail) {
  constexpr int PER = 16 / sizeof(T);
  extern __shared__ float xin[];                   // [n_in], then the partial sums [NT * PER]
  float* red = xin + n_in;
  const T* ip = in + blockIdx.x * in_row + blockIdx.y * in_head;
  T* op = out + blockIdx.x * out_row + blockIdx.y * out_head;
  const T* wp = w + static_cast<int64_t>(blockIdx.y) * n_in * n_out;
  const int tid = threadIdx.x;
  for (int i = tid; i < n_in; i += NT) xin[i] = to_f32(ip[i]);
  for (int jb = 0; jb < n_out; jb += NT * PER) {
    const int jn = min(n_out - jb, NT * PER);
    const int JC = jn / PER, IS = NT / JC;
    const int jc = tid % JC, is = tid / JC;
    float acc[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) acc[u] = 0.f;
    __syncthreads();                               // xin is there; red is free
    if (is < IS) {
      const T* col = wp + jb + jc * PER;
#pragma unroll 8
      for (int i = is; i < n_in; i += IS) {
        const uint4 raw = *reinterpret_cast<const uint4*>(col + static_cast<int64_t>(i) * n_out);
        const float x = xin[i];
        if constexpr (sizeof(T) == 2) {
          const unsigned u4[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            acc[2 * u] += x * __uint_as_float(u4[u] << 16);
            acc[2 * u + 1] += x * __uint_as_float(u4[u] & 0xFFFF0000u);
          }
        } else {
          acc[0] += x * __uint_as_float(raw.x); acc[1] += x * __uint_as_float(raw.y);
          acc[2] += x * __uint_as_float(raw.z); acc[3] += x * __uint_as_float(raw.w);
        }
      }
#pragma unroll
      for (int u = 0; u < PER; ++u) red[is * jn + jc * PER + u] = acc[u];
    }
    __syncthreads();
    for (int j = tid; j < jn; j += NT) {
      float s = 0.f;
      for (int k = 0; k < IS; ++k) s += red[k * jn + j];
      op[jb + j] = from_f32<T>(s);
    }
  }
  for (int c = tid; c < n_tail; c += NT) op[n_out + c] = ip[n_in + c];
}

__device__ __forceinline__ float activation(float v, int kind) {
  if (kind == GBXM_ACT_RELU2) { const float r = fmaxf(v, 0.f); return r * r; }
  return 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
}

template <typename T>
__global__ __launch_bounds__(NT) void activate_kernel(T* __restrict__ z, int64_t n, int kind) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x;
  if (i >= n) return;
  z[i] = from_f32<T>(activation(to_f32(z[i]), kind));
}

// 16 bytes per thread (n a multiple of the vector, base 16-byte aligned)
template <typename T>
__global__ __launch_bounds__(NT) void activate_vec_kernel(T* __restrict__ z, int64_t n_vec, int kind) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x;
  if (i >= n_vec) return;
  uint4* p = reinterpret_cast<uint4*>(z) + i;
  uint4 raw = *p;
  unsigned u[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if constexpr (sizeof(T) == 2) {
      const float lo = activation(__uint_as_float(u[k] << 16), kind), hi = activation(__uint_as_float(u[k] & 0xFFFF0000u), kind);
      u[k] = static_cast<unsigned>(f32_to_bf16(lo)) | (static_cast<unsigned>(f32_to_bf16(hi)) << 16);
    } else {
      u[k] = __float_as_uint(activation(__uint_as_float(u[k]), kind));
    }
  }
  *p = uint4{u[0], u[1], u[2], u[3]};
}

template <typename T>
__global__ __launch_bounds__(NT) void slot_append_kernel(const T* __restrict__ k, int64_t k_stride, int k_width, const T* __restrict__ v,
                                                        int64_t v_stride, int v_width, T* __restrict__ kc, T* __restrict__ vc,
                                                        const int* __restrict__ seq, const int* __restrict__ tok, int keep, int ring) {
  const int64_t t = blockIdx.x;
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], n = seq[4 * b + 2];
  if (pos >= keep && pos + ring < pos0 + n) return;      // a later row of this step takes the same ring row
  const int64_t row = static_cast<int64_t>(slot) * (keep + ring) + (pos < keep ? pos : keep + (pos - keep) % ring);
  for (int c = threadIdx.x; c < k_width; c += NT) kc[row * k_width + c] = k[t * k_stride + c];
  if (v)
    for (int c = threadIdx.x; c < v_width; c += NT) vc[row * v_width + c] = v[t * v_stride + c];
}

bool act_ok(int act) { return act == GBXM_BF16 || act == GBXM_F32; }

}  // namespace

int launch_sink_tiles(const gbxm_sink_attn_args& a, hipStream_t s);     // mixers_sink_mfma.hip; GBXM_ERR_UNSUPPORTED: not its shape
int launch_sink_group(const gbxm_sink_attn_args& a, hipStream_t s);     // the same for steps of single rows
bool sink_tiles_shape(int dk, int dv);

int launch_sink_reduce(const gbxm_sink_attn_args& a, int splits, hipStream_t s) {
  sink_reduce_kernel<bf16_t, true><<<dim3(a.T, a.H), 256, 0, s>>>(static_cast<const float*>(a.partial), static_cast<bf16_t*>(a.out), a.sink,
                                                                  static_cast<const bf16_t*>(a.gate), a.gate_row, a.T, a.H, a.dv, splits);
  return after_launch("sink_attention (join of key splits)");
}

}  // namespace gbxm

using namespace gbxm;

#define GBXM_DISPATCH(act, CALL)              \
  do {                                        \
    if ((act) == GBXM_BF16) { using T = bf16_t; CALL; } else { using T = float; CALL; } \
  } while (0)

extern "C" {

int gbxm_stream_add(float* x, const void* a, const void* b, int64_t n, int32_t act, void* stream) {
  if (!act_ok(act) || !x || !a || n < 0) return fail(GBXM_ERR_INVALID, "stream_add: bad argument");
  if (n == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (stream_add_kernel<T><<<dim3((n + NT - 1) / NT), NT, 0, s>>>(x, static_cast<const T*>(a), static_cast<const T*>(b), n)));
  return after_launch("stream_add");
}

int gbxm_stream_add_norm(float* x, const void* a, const void* b, const float* w, void* h, int64_t T_, int32_t width, float eps, int32_t act,
                         void* stream) {
  if (!act_ok(act) || !x || !a || !w || !h || T_ < 0 || width <= 0) return fail(GBXM_ERR_INVALID, "stream_add_norm: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (stream_add_norm_kernel<T><<<dim3(T_), NT, 0, s>>>(x, static_cast<const T*>(a), static_cast<const T*>(b), w, static_cast<T*>(h),
                                                                          width, eps)));
  return after_launch("stream_add_norm");
}

int gbxm_head_project(const void* in, int64_t in_row, int64_t in_head, const void* w, void* out, int64_t out_row, int64_t out_head, int64_t T_,
                      int32_t H, int32_t n_in, int32_t n_out, int32_t n_tail, int32_t act, void* stream) {
  if (!act_ok(act) || !in || !w || !out || T_ < 0 || H < 1 || H > 65535 || n_in < 1 || n_out < 1 || n_tail < 0)
    return fail(GBXM_ERR_INVALID, "head_project: bad argument");
  if (n_in > 12 * 1024) return fail(GBXM_ERR_UNSUPPORTED, "head_project: %d input channels per head", n_in);
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int per = act == GBXM_BF16 ? 8 : 4;
  if (n_out % per == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0) {
    GBXM_DISPATCH(act, (head_project_vec_kernel<T><<<dim3(T_, H), NT, (n_in + NT * per) * sizeof(float), s>>>(
                           static_cast<const T*>(in), in_row, in_head, static_cast<const T*>(w), static_cast<T*>(out), out_row, out_head, n_in, n_out,
                           n_tail)));
    return after_launch("head_project");
  }
  GBXM_DISPATCH(act, (head_project_kernel<T><<<dim3(T_, H), NT, n_in * sizeof(float), s>>>(static_cast<const T*>(in), in_row, in_head,
                                                                                           static_cast<const T*>(w), static_cast<T*>(out), out_row,
                                                                                           out_head, n_in, n_out, n_tail)));
  return after_launch("head_project");
}

int gbxm_activate(void* z, int64_t n, int32_t kind, int32_t act, void* stream) {
  if (!act_ok(act) || !z || n < 0 || (kind != GBXM_ACT_RELU2 && kind != GBXM_ACT_GELU_TANH)) return fail(GBXM_ERR_INVALID, "activate: bad argument");
  if (n == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int per = act == GBXM_BF16 ? 8 : 4;
  if (n % per == 0 && reinterpret_cast<uintptr_t>(z) % 16 == 0) {
    const int64_t nv = n / per;
    GBXM_DISPATCH(act, (activate_vec_kernel<T><<<dim3((nv + NT - 1) / NT), NT, 0, s>>>(static_cast<T*>(z), nv, kind)));
    return after_launch("activate");
  }
  GBXM_DISPATCH(act, (activate_kernel<T><<<dim3((n + NT - 1) / NT), NT, 0, s>>>(static_cast<T*>(z), n, kind)));
  return after_launch("activate");
}

int gbxm_rotate_norm_heads(void* rows, int64_t T_, int64_t row_stride, const int32_t* positions, int64_t pos_stride, const gbxm_head_segment* segs,
                           int32_t n_segs, float eps, int32_t act, void* stream) {
  if (!act_ok(act) || !rows || !positions || !segs || n_segs < 1 || n_segs > GBXM_MAX_SEGMENTS || T_ < 0)
    return fail(GBXM_ERR_INVALID, "rotate_norm_heads: bad argument");
  Segments sg{};
  int max_dim = 0;
  for (int i = 0; i < n_segs; ++i) {
    const gbxm_head_segment& g = segs[i];
    if (g.offset < 0 || g.heads < 1 || g.head_dim < 1 || g.offset + static_cast<int64_t>(g.heads) * g.head_dim > row_stride || g.rot_dims < 0 ||
        g.rot_dims % 2 || g.rot_offset < 0 || g.rot_offset + g.rot_dims > g.head_dim || (g.rot_dims && !g.freq) || g.norm < 0 || g.norm > 4 ||
        ((g.norm == 2 || g.norm == 4) && !g.weight))
      return fail(GBXM_ERR_INVALID, "rotate_norm_heads: segment %d does not fit its rows", i);
    sg.s[i] = g;
    max_dim = std::max(max_dim, g.head_dim);
  }
  const size_t lds = (static_cast<size_t>(NW) * 2 * max_dim + 2 * (max_dim / 2 + 1)) * sizeof(float);
  if (lds > 60 * 1024) return fail(GBXM_ERR_UNSUPPORTED, "rotate_norm_heads: heads of %d channels", max_dim);
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (rotate_norm_kernel<T><<<dim3(T_, n_segs), NT, lds, s>>>(static_cast<T*>(rows), row_stride, positions, pos_stride, sg, eps, max_dim)));
  return after_launch("rotate_norm_heads");
}

int gbxm_slot_append(const void* k, int64_t k_stride, int32_t k_width, const void* v, int64_t v_stride, int32_t v_width, void* kcache, void* vcache,
                     const int32_t* seq, const int32_t* tok, int64_t T_, int32_t keep, int32_t ring, int32_t act, void* stream) {
  if (!act_ok(act) || !k || !kcache || !seq || !tok || k_width <= 0 || k_stride < k_width || keep < 0 || ring < 1 || T_ < 0 ||
      (v && (!vcache || v_width <= 0 || v_stride < v_width)))
    return fail(GBXM_ERR_INVALID, "slot_append: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (slot_append_kernel<T><<<dim3(T_), NT, 0, s>>>(static_cast<const T*>(k), k_stride, k_width, static_cast<const T*>(v), v_stride,
                                                                      v_width, static_cast<T*>(kcache), static_cast<T*>(vcache), seq, tok, keep, ring)));
  return after_launch("slot_append");
}

int gbxm_sink_attention_tiled(int32_t dk, int32_t dv, int32_t act, int32_t decode_only) {
  return act == GBXM_BF16 && sink_tiles_shape(dk, dv);          // (steps of single rows: the grouped form of the same products)
}

int gbxm_sink_attention(const gbxm_sink_attn_args* a, void* stream) {
  if (!a || !a->q || !a->k_new || !a->v_new || !a->seq || !a->tok || !a->out) return fail(GBXM_ERR_INVALID, "sink_attention: null argument");
  if (!act_ok(a->act)) return fail(GBXM_ERR_INVALID, "sink_attention: dtype");
  if (a->H <= 0 || a->G <= 0 || a->H % a->G || a->dk <= 0 || a->dv <= 0 || a->keep < 0 || a->ring < 1 || a->T < 0 || a->B < 0 ||
      (a->kcache && !a->vcache))
    return fail(GBXM_ERR_INVALID, "sink_attention: bad geometry");
  if (a->window > 0 && a->ring < a->window) return fail(GBXM_ERR_INVALID, "sink_attention: a ring shorter than the window");
  if (a->T == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!a->decode_only && a->act == GBXM_BF16 && a->tiles && a->n_tiles > 0) {
    const int rc = launch_sink_tiles(*a, s);
    if (rc != GBXM_ERR_UNSUPPORTED) return rc;
  }
  if (a->decode_only && a->act == GBXM_BF16 && a->H <= 65535) {
    const int rc = launch_sink_group(*a, s);
    if (rc != GBXM_ERR_UNSUPPORTED) return rc;
  }
  SinkGeo g{a->H, a->G, a->dk, a->dv, a->window, a->keep, a->ring, a->scale, a->q_row, a->q_head, a->k_row, a->k_head, a->v_row, a->v_head,
            a->kc_slot, a->kc_row, a->kc_head, a->vc_slot, a->vc_row, a->vc_head, a->gate_row};
  const int R = a->H / a->G;
  if (a->dv > NCH * DCH) return fail(GBXM_ERR_UNSUPPORTED, "sink_attention: value size %d beyond the row kernel (%d)", a->dv, NCH * DCH);
  auto lds_of = [&](int rc_) {
    return static_cast<size_t>(2 * KT) * sizeof(void*) + static_cast<size_t>(rc_) * (a->dk + KT + 3 + NW * a->dv) * sizeof(float);
  };
  int rc = R < RC ? R : RC;
  while (rc > 1 && lds_of(rc) > 60 * 1024) --rc;
  if (lds_of(rc) > 60 * 1024) return fail(GBXM_ERR_UNSUPPORTED, "sink_attention: head sizes dk=%d dv=%d are beyond the row kernel", a->dk, a->dv);
  const int chunks = (R + rc - 1) / rc;
  if (a->T > 0x7fffffffLL || a->G * chunks > 65535 || a->H > 65535) return fail(GBXM_ERR_UNSUPPORTED, "sink_attention: grid");
  return a->act == GBXM_BF16 ? launch_rows<bf16_t, true>(*a, g, rc, chunks, lds_of(rc), s) : launch_rows<float, false>(*a, g, rc, chunks, lds_of(rc), s);
}

}  // extern "C"
