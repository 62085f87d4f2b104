// Grouped matrix-core products of routed experts for bf16 prompt portions (mechanism: mixers_moe.hip).
//
// 1. expert_sort_kernel: the step's (row, choice) pairs counted and bucketed by expert on the device (one workgroup, LDS counters):
//    offsets[E + 1], the pair ids in expert order, and the table of row tiles (expert, first pair) the two products walk.  Nothing
//    returns to the host.
// 2. expert_up_kernel:   act[p] = silu(gate_e h) * (up_e h) for the pairs of expert e, 128 pairs x 128 hidden channels per workgroup;
// 3. expert_down_kernel: y[pair] = down_e act[p], 128 pairs x 256 output channels per workgroup.
// Products are computed swapped -- C^T[channel, pair] = mfma(weight rows, activation rows) -- so a lane ends up with four consecutive
// channels of one pair (8-byte stores) and the gate / up pair of a channel sits in the same lane for the activation.
// Weight fragments are 16-byte loads straight from the row-major matrices (every wave has rows of its own); the activation tile,
// which all four waves share, goes global -> registers (one chunk ahead) -> LDS once per workgroup: counters showed the version
// in which every wave fetched it for itself waiting on L2 -> L1 traffic for more than half of its cycles.
// The contraction runs in chunks of 64 elements (a 32-element tail when the size is not a multiple of 64); inside a chunk the lane
// half hb takes the contiguous half [hb * C/2, (hb + 1) * C/2) and feeds it to the chunk's MFMA steps 8 elements at a time -- the
// order of the contraction is free as long as both operands use the same one -- so a lane reads 64 contiguous bytes per chunk.
// The grid is sized for the worst case sum_e ceil(n_e / 128) <= P / 128 + E; surplus workgroups leave at once.
#include <type_traits>
#include "mixers_mfma.h"

namespace gbxm {
namespace {

constexpr int RT = 128;         // pairs per workgroup tile
constexpr int BROW = 128 + 16;  // LDS bytes per activation row of a chunk (+16: conflict-free 16-byte fragment reads)

__global__ __launch_bounds__(1024) void expert_sort_kernel(const int* __restrict__ idx, int* __restrict__ offsets, int* __restrict__ sorted,
                                                          int* __restrict__ tile_tab, int n_tiles, int P, int E) {
  extern __shared__ int sm[];                 // counts [E] | cursor [E] | first tile [E]
  int* counts = sm;
  int* cursor = sm + E;
  int* first = sm + 2 * E;
  for (int e = threadIdx.x; e < E; e += 1024) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < P; i += 1024) atomicAdd(&counts[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      offsets[e] = run; cursor[e] = run; first[e] = tiles;
      run += counts[e];
      tiles += (counts[e] + RT - 1) / RT;
    }
    offsets[E] = run;
    sm[3 * E] = tiles;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < P; i += 1024) sorted[atomicAdd(&cursor[idx[i]], 1)] = i;
  for (int e = threadIdx.x; e < E; e += 1024) {
    const int nt = (counts[e] + RT - 1) / RT, lo = offsets[e];
    for (int t = 0; t < nt; ++t) { tile_tab[2 * (first[e] + t)] = e; tile_tab[2 * (first[e] + t) + 1] = lo + t * RT; }
  }
  for (int t = sm[3 * E] + threadIdx.x; t < n_tiles; t += 1024) tile_tab[2 * t] = -1;
}

// Workgroup ids go round-robin over the 8 XCDs, each with an L2 of its own: row tile = (id % 8) * (gridDim.x / 8) + id / 8 gives every
// XCD a contiguous run of row tiles, so the row tiles of ONE expert, which read the same weights, run on one XCD next to each other.
// (gridDim.x is a multiple of 8.)
__device__ __forceinline__ int xcd_row_tile() { return (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8; }

// Activation tile of a chunk: 128 rows x C elements.  Thread t moves the 16-byte pieces t + 256 i (i < 4): row = piece / 8, column piece
// = piece % 8 (only the first C / 8 column pieces exist in a 32-element tail).
struct BTile {
  const bf16_t* rowp[4];      // this thread's four rows (already offset by its column piece)
  int lds_off[4];
  int cpiece;
  u32x4 regs[4];
  __device__ __forceinline__ void fetch(int k0, int pieces) {
#pragma unroll
    for (int i = 0; i < 4; ++i) regs[i] = cpiece < pieces ? *reinterpret_cast<const u32x4*>(rowp[i] + k0) : u32x4{0, 0, 0, 0};
  }
  __device__ __forceinline__ void park(unsigned char* bl) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(bl + lds_off[i]) = regs[i];
  }
};

__global__ __launch_bounds__(256) void expert_up_kernel(const bf16_t* __restrict__ h, const bf16_t* __restrict__ gate_up, const int* __restrict__ offsets,
                                                       const int* __restrict__ sorted, const int* __restrict__ tile_tab, bf16_t* __restrict__ act,
                                                       int K, int F, int top, int kind, float limit) {
  __shared__ __attribute__((aligned(16))) unsigned char bl[RT * BROW];
  const int bt = xcd_row_tile();
  const int e = tile_tab[2 * bt];
  if (e < 0) return;                                                  // (workgroup-uniform)
  const int lo = tile_tab[2 * bt + 1], hi = offsets[e + 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hb = lane >> 5;
  const int f0 = blockIdx.y * 128 + wave * 32;
  const bool live = f0 < F;                                           // a wave past the last channel still moves its share of the tile
  const bf16_t* wgl = gate_up + (static_cast<int64_t>(e) * 2 * F + (live ? f0 + r : 0)) * K;
  const bf16_t* wul = wgl + static_cast<int64_t>(F) * K;
  BTile b;
  b.cpiece = tid & 7;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = (tid >> 3) + 32 * i;
    b.rowp[i] = h + static_cast<int64_t>(sorted[min(lo + row, hi - 1)] / top) * K + b.cpiece * 8;
    b.lds_off[i] = row * BROW + b.cpiece * 16;
  }
  f32x16 ag[4], au[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) { ag[j] = f32x16{0}; au[j] = f32x16{0}; }

  auto chunk = [&](int k0, auto steps_c) {
    constexpr int S = decltype(steps_c)::value;                         // MFMA steps of the chunk: 4 (64 elements) or 2 (32)
    const int off = k0 + hb * (S * 8);
    u32x4 fg[S], fu[S];                                                 // weight fragments: requested ahead of the tile hand-over
#pragma unroll
    for (int i = 0; i < S; ++i) {
      fg[i] = *reinterpret_cast<const u32x4*>(wgl + off + i * 8);
      fu[i] = *reinterpret_cast<const u32x4*>(wul + off + i * 8);
    }
    __syncthreads();                                                    // the previous chunk's fragments have been read
    b.park(bl);
    __syncthreads();
    const int kn = k0 + S * 16;
    if (kn < K) b.fetch(kn, kn + 64 <= K ? 8 : 4);                      // the next chunk travels while this one is multiplied
    if (!live) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x4 fb[S];
#pragma unroll
      for (int i = 0; i < S; ++i) fb[i] = *reinterpret_cast<const u32x4*>(bl + (j * 32 + r) * BROW + hb * (S * 16) + i * 16);
#pragma unroll
      for (int i = 0; i < S; ++i) {
        ag[j] = mfma_bf16(fg[i], fb[i], ag[j]);
        au[j] = mfma_bf16(fu[i], fb[i], au[j]);
      }
    }
  };
  b.fetch(0, K >= 64 ? 8 : 4);
  int k0 = 0;
  for (; k0 + 64 <= K; k0 += 64) chunk(k0, std::integral_constant<int, 4>{});
  if (k0 < K) chunk(k0, std::integral_constant<int, 2>{});
  if (!live) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = lo + j * 32 + r;
    if (row >= hi) continue;
    bf16_t* ap = act + static_cast<int64_t>(row) * F + f0 + 4 * hb;
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { const float g = ag[j][4 * q4 + i]; v[i] = glu_act<true>(g, au[j][4 * q4 + i], kind, limit, 1.702f); }
      *reinterpret_cast<u32x2*>(ap + 8 * q4) = u32x2{pack2(v[0], v[1]), pack2(v[2], v[3])};
    }
  }
}

__global__ __launch_bounds__(256) void expert_down_kernel(const bf16_t* __restrict__ act, const bf16_t* __restrict__ down, const int* __restrict__ offsets,
                                                         const int* __restrict__ sorted, const int* __restrict__ tile_tab, bf16_t* __restrict__ y,
                                                         int K, int F) {
  __shared__ __attribute__((aligned(16))) unsigned char bl[RT * BROW];
  const int bt = xcd_row_tile();
  const int e = tile_tab[2 * bt];
  if (e < 0) return;
  const int lo = tile_tab[2 * bt + 1], hi = offsets[e + 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hb = lane >> 5;
  const int c0 = blockIdx.y * 256 + wave * 64;
  const bool live = c0 < K;
  const bool second = c0 + 32 < K;                                    // K is a multiple of 32: the wave's second channel block may not exist
  const bf16_t* wl[2];
  wl[0] = down + (static_cast<int64_t>(e) * K + (live ? c0 + r : 0)) * F;
  wl[1] = second ? wl[0] + static_cast<int64_t>(32) * F : wl[0];
  BTile b;
  b.cpiece = tid & 7;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = (tid >> 3) + 32 * i;
    b.rowp[i] = act + static_cast<int64_t>(min(lo + row, hi - 1)) * F + b.cpiece * 8;
    b.lds_off[i] = row * BROW + b.cpiece * 16;
  }
  f32x16 acc[2][4];
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[c][j] = f32x16{0};

  auto chunk = [&](int f0_, auto steps_c) {
    constexpr int S = decltype(steps_c)::value;
    const int off = f0_ + hb * (S * 8);
    u32x4 fa[2][S];
#pragma unroll
    for (int i = 0; i < S; ++i) {
      fa[0][i] = *reinterpret_cast<const u32x4*>(wl[0] + off + i * 8);
      fa[1][i] = *reinterpret_cast<const u32x4*>(wl[1] + off + i * 8);
    }
    __syncthreads();
    b.park(bl);
    __syncthreads();
    const int fn = f0_ + S * 16;
    if (fn < F) b.fetch(fn, fn + 64 <= F ? 8 : 4);
    if (!live) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x4 fb[S];
#pragma unroll
      for (int i = 0; i < S; ++i) fb[i] = *reinterpret_cast<const u32x4*>(bl + (j * 32 + r) * BROW + hb * (S * 16) + i * 16);
#pragma unroll
      for (int i = 0; i < S; ++i) {
        acc[0][j] = mfma_bf16(fa[0][i], fb[i], acc[0][j]);
        acc[1][j] = mfma_bf16(fa[1][i], fb[i], acc[1][j]);
      }
    }
  };
  b.fetch(0, F >= 64 ? 8 : 4);
  int fc = 0;
  for (; fc + 64 <= F; fc += 64) chunk(fc, std::integral_constant<int, 4>{});
  if (fc < F) chunk(fc, std::integral_constant<int, 2>{});
  if (!live) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = lo + j * 32 + r;
    if (row >= hi) continue;
    bf16_t* yp = y + static_cast<int64_t>(sorted[row]) * K + c0 + 4 * hb;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (c == 1 && !second) continue;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        *reinterpret_cast<u32x2*>(yp + c * 32 + 8 * q4) =
            u32x2{pack2(acc[c][j][4 * q4], acc[c][j][4 * q4 + 1]), pack2(acc[c][j][4 * q4 + 2], acc[c][j][4 * q4 + 3])};
    }
  }
}

size_t align16(size_t n) { return (n + 15) & ~static_cast<size_t>(15); }
constexpr int64_t MIN_PAIRS = 256;        // below this the weight-streaming row kernels read less
int tiles_of(int64_t P, int E) { return static_cast<int>((P / RT + E + 7) / 8 * 8); }

}  // namespace

size_t expert_grouped_workspace(int64_t T, int K, int F, int E, int top) {
  const int64_t P = T * top;
  if (P < MIN_PAIRS || K % 32 || F % 32 || E > 4096 || P > 0x3fffffff) return 0;
  return align16(sizeof(int) * (E + 1)) + align16(sizeof(int) * P) + align16(sizeof(int) * 2 * tiles_of(P, E)) + align16(sizeof(bf16_t) * P * F);
}

int launch_expert_grouped(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T, int K, int F, int E, int top,
                          int kind, float limit, void* ws, size_t ws_bytes, hipStream_t s) {
  const size_t need = expert_grouped_workspace(T, K, F, E, top);
  if (need == 0) return GBXM_ERR_UNSUPPORTED;
  if (ws_bytes < need) return fail(GBXM_ERR_INVALID, "expert_glu: workspace of %zu bytes, %zu needed", ws_bytes, need);
  if ((reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(down) | reinterpret_cast<uintptr_t>(y) |
       reinterpret_cast<uintptr_t>(ws)) % 16)
    return GBXM_ERR_UNSUPPORTED;
  const int P = static_cast<int>(T * top);
  const int tiles = tiles_of(P, E);
  unsigned char* w = static_cast<unsigned char*>(ws);
  int* offsets = reinterpret_cast<int*>(w);
  w += align16(sizeof(int) * (E + 1));
  int* sorted = reinterpret_cast<int*>(w);
  w += align16(sizeof(int) * P);
  int* tile_tab = reinterpret_cast<int*>(w);
  w += align16(sizeof(int) * 2 * tiles);
  bf16_t* act = reinterpret_cast<bf16_t*>(w);
  expert_sort_kernel<<<1, 1024, (3 * E + 1) * sizeof(int), s>>>(idx, offsets, sorted, tile_tab, tiles, P, E);
  expert_up_kernel<<<dim3(tiles, (F + 127) / 128), 256, 0, s>>>(static_cast<const bf16_t*>(h), static_cast<const bf16_t*>(gate_up), offsets, sorted,
                                                                 tile_tab, act, K, F, top, kind, limit);
  expert_down_kernel<<<dim3(tiles, (K + 255) / 256), 256, 0, s>>>(act, static_cast<const bf16_t*>(down), offsets, sorted, tile_tab,
                                                                   static_cast<bf16_t*>(y), K, F);
  return after_launch("expert_glu (grouped)");
}

}  // namespace gbxm
