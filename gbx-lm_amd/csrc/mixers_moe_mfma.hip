// Grouped matrix-core products of routed experts for bf16 prompt portions (mechanism: mixers_moe.hip).
//
// 1. expert_sort_kernel: the step's (row, choice) pairs counted and bucketed by expert on the device (one workgroup, LDS counters):
//    offsets[E + 1] and the pair ids in expert order.  Nothing returns to the host.
// 2. expert_up_kernel:   act[p] = silu(gate_e h) * (up_e h) for the pairs of expert e, 64 pairs x 128 hidden channels per workgroup;
// 3. expert_down_kernel: y[pair] = down_e act[p], 64 pairs x 256 output channels per workgroup.
// Products are computed swapped -- C^T[channel, pair] = mfma(weight rows, activation rows) -- so both operands are 16-byte
// fragments straight from their row-major matrices (contraction index contiguous), a lane ends up with four consecutive
// channels of one pair (8-byte stores), and the gate / up pair of a channel sits in the same lane for the activation.
// Operands come from global memory through L1 / L2 (a wave's 64 x 64 tile: four 16-byte loads per four MFMAs); the grid is sized
// for the worst case sum_e ceil(n_e / 64) <= P / 64 + E and surplus workgroups leave at once.
#include "mixers_mfma.h"

namespace gbxm {
namespace {

constexpr int RT = 64;          // pairs per workgroup tile

__global__ __launch_bounds__(1024) void expert_sort_kernel(const int* __restrict__ idx, int* __restrict__ offsets, int* __restrict__ sorted, int P,
                                                          int E) {
  extern __shared__ int sm[];                 // counts [E] | cursor [E]
  int* counts = sm;
  int* cursor = sm + E;
  for (int e = threadIdx.x; e < E; e += 1024) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < P; i += 1024) atomicAdd(&counts[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) { offsets[e] = run; cursor[e] = run; run += counts[e]; }
    offsets[E] = run;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < P; i += 1024) sorted[atomicAdd(&cursor[idx[i]], 1)] = i;
}

// (expert, first pair, end) of row tile `bt`, or expert -1
__device__ __forceinline__ void find_tile(const int* __restrict__ offsets, int E, int bt, int& e_out, int& lo, int& hi) {
  int seen = 0;
  e_out = -1;
  for (int e = 0; e < E; ++e) {
    const int a = offsets[e], b = offsets[e + 1];
    const int nt = (b - a + RT - 1) / RT;
    if (bt < seen + nt) { e_out = e; lo = a + (bt - seen) * RT; hi = b; return; }
    seen += nt;
  }
}

__global__ __launch_bounds__(256) void expert_up_kernel(const bf16_t* __restrict__ h, const bf16_t* __restrict__ gate_up, const int* __restrict__ offsets,
                                                       const int* __restrict__ sorted, bf16_t* __restrict__ act, int K, int F, int E, int top) {
  int e, lo, hi;
  find_tile(offsets, E, blockIdx.x, e, lo, hi);
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, hb = lane >> 5;
  const int f0 = blockIdx.y * 128 + wave * 32;
  if (f0 >= F) return;
  const bf16_t* wg = gate_up + (static_cast<int64_t>(e) * 2 * F + f0 + r) * K + hb * 8;
  const bf16_t* wu = wg + static_cast<int64_t>(F) * K;
  const bf16_t* hp[2];
  int row[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    row[j] = lo + j * 32 + r;
    hp[j] = h + static_cast<int64_t>(sorted[min(row[j], hi - 1)] / top) * K + hb * 8;
  }
  f32x16 ag[2], au[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) { ag[j] = f32x16{0}; au[j] = f32x16{0}; }
  for (int k = 0; k < K; k += 16) {
    const u32x4 a_g = *reinterpret_cast<const u32x4*>(wg + k), a_u = *reinterpret_cast<const u32x4*>(wu + k);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const u32x4 b = *reinterpret_cast<const u32x4*>(hp[j] + k);
      ag[j] = mfma_bf16(a_g, b, ag[j]);
      au[j] = mfma_bf16(a_u, b, au[j]);
    }
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (row[j] >= hi) continue;
    bf16_t* ap = act + static_cast<int64_t>(row[j]) * F + f0 + 4 * hb;
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { const float g = ag[j][4 * q4 + i]; v[i] = g * sigmoid_<true>(g) * au[j][4 * q4 + i]; }
      *reinterpret_cast<u32x2*>(ap + 8 * q4) = u32x2{pack2(v[0], v[1]), pack2(v[2], v[3])};
    }
  }
}

__global__ __launch_bounds__(256) void expert_down_kernel(const bf16_t* __restrict__ act, const bf16_t* __restrict__ down, const int* __restrict__ offsets,
                                                         const int* __restrict__ sorted, bf16_t* __restrict__ y, int K, int F, int E) {
  int e, lo, hi;
  find_tile(offsets, E, blockIdx.x, e, lo, hi);
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, hb = lane >> 5;
  const int c0 = blockIdx.y * 256 + wave * 64;
  if (c0 >= K) return;
  const bool second = c0 + 32 < K;                                    // K is a multiple of 32: the wave's second channel block may not exist
  const bf16_t* wd[2];
  wd[0] = down + (static_cast<int64_t>(e) * K + c0 + r) * F + hb * 8;
  wd[1] = second ? wd[0] + static_cast<int64_t>(32) * F : wd[0];
  const bf16_t* ap[2];
  int row[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    row[j] = lo + j * 32 + r;
    ap[j] = act + static_cast<int64_t>(min(row[j], hi - 1)) * F + hb * 8;
  }
  f32x16 acc[2][2];
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[c][j] = f32x16{0};
  for (int f = 0; f < F; f += 16) {
    const u32x4 a0 = *reinterpret_cast<const u32x4*>(wd[0] + f), a1 = *reinterpret_cast<const u32x4*>(wd[1] + f);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const u32x4 b = *reinterpret_cast<const u32x4*>(ap[j] + f);
      acc[0][j] = mfma_bf16(a0, b, acc[0][j]);
      acc[1][j] = mfma_bf16(a1, b, acc[1][j]);
    }
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (row[j] >= hi) continue;
    bf16_t* yp = y + static_cast<int64_t>(sorted[row[j]]) * K + c0 + 4 * hb;
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
constexpr int64_t MIN_PAIRS = 256;        // below this the weight-streaming row kernel reads less

}  // namespace

size_t expert_grouped_workspace(int64_t T, int K, int F, int E, int top) {
  const int64_t P = T * top;
  if (P < MIN_PAIRS || K % 32 || F % 32 || E > 4096 || P > 0x3fffffff) return 0;
  return align16(sizeof(int) * (E + 1)) + align16(sizeof(int) * P) + align16(sizeof(bf16_t) * P * F);
}

int launch_expert_grouped(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T, int K, int F, int E, int top,
                          void* ws, size_t ws_bytes, hipStream_t s) {
  const size_t need = expert_grouped_workspace(T, K, F, E, top);
  if (need == 0) return GBXM_ERR_UNSUPPORTED;
  if (ws_bytes < need) return fail(GBXM_ERR_INVALID, "expert_glu: workspace of %zu bytes, %zu needed", ws_bytes, need);
  if ((reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(down) | reinterpret_cast<uintptr_t>(y) |
       reinterpret_cast<uintptr_t>(ws)) % 16)
    return GBXM_ERR_UNSUPPORTED;
  const int P = static_cast<int>(T * top);
  unsigned char* w = static_cast<unsigned char*>(ws);
  int* offsets = reinterpret_cast<int*>(w);
  int* sorted = reinterpret_cast<int*>(w + align16(sizeof(int) * (E + 1)));
  bf16_t* act = reinterpret_cast<bf16_t*>(w + align16(sizeof(int) * (E + 1)) + align16(sizeof(int) * P));
  expert_sort_kernel<<<1, 1024, 2 * E * sizeof(int), s>>>(idx, offsets, sorted, P, E);
  const int tiles = P / RT + E;
  expert_up_kernel<<<dim3(tiles, (F + 127) / 128), 256, 0, s>>>(static_cast<const bf16_t*>(h), static_cast<const bf16_t*>(gate_up), offsets, sorted, act,
                                                                 K, F, E, top);
  expert_down_kernel<<<dim3(tiles, (K + 255) / 256), 256, 0, s>>>(act, static_cast<const bf16_t*>(down), offsets, sorted, static_cast<bf16_t*>(y), K, F, E);
  return after_launch("expert_glu (grouped)");
}

}  // namespace gbxm
