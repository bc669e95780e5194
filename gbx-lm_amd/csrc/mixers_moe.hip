// Routed gated MLPs over dense stacked experts:  y[t][s] = down_e (silu(gate_e h_t) * (up_e h_t)),  e = idx[t][s].
//
//   * expert_rows_kernel -- one workgroup per (row, chosen expert): the row in LDS, a wave per output channel with its lanes
//     across the contraction (coalesced weight reads, fp32 sums in a fixed order).  Weight-bandwidth bound: the kernel of decode
//     steps, of fp32 models and of shapes the grouped kernel does not take.
//   * grouped matrix-core products for bf16 prompt portions (rows sorted by expert on the device, no host round trip).
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256, NW = NT / 64;

template <typename T, bool FAST>
__global__ __launch_bounds__(NT) void expert_rows_kernel(const T* __restrict__ h, const T* __restrict__ gate_up, const T* __restrict__ down,
                                                        const int* __restrict__ idx, T* __restrict__ y, int K, int F, int top) {
  extern __shared__ float lds[];                    // row [K] | act [F]
  float* hl = lds;
  float* al = lds + K;
  const int64_t pair = blockIdx.x;                  // t * top + s
  const int e = idx[pair];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* hr = h + (pair / top) * K;
  for (int k = threadIdx.x; k < K; k += NT) hl[k] = to_f32(hr[k]);
  __syncthreads();
  const T* wg = gate_up + static_cast<int64_t>(e) * 2 * F * K;
  const T* wu = wg + static_cast<int64_t>(F) * K;
  for (int f = wave; f < F; f += NW) {
    const T* g = wg + static_cast<int64_t>(f) * K;
    const T* u = wu + static_cast<int64_t>(f) * K;
    float ag = 0.f, au = 0.f;
    for (int k = lane; k < K; k += 64) { const float x = hl[k]; ag += to_f32(g[k]) * x; au += to_f32(u[k]) * x; }
    ag = wave_sum(ag); au = wave_sum(au);
    if (lane == 0) al[f] = to_f32(from_f32<T>(ag * sigmoid_<FAST>(ag) * au));   // the hidden row is an activation: rounded as one
  }
  __syncthreads();
  const T* wd = down + static_cast<int64_t>(e) * K * F;
  T* yr = y + pair * K;
  for (int c = wave; c < K; c += NW) {
    const T* d = wd + static_cast<int64_t>(c) * F;
    float acc = 0.f;
    for (int f = lane; f < F; f += 64) acc += to_f32(d[f]) * al[f];
    acc = wave_sum(acc);
    if (lane == 0) yr[c] = from_f32<T>(acc);
  }
}

}  // namespace

int launch_expert_grouped(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T, int K, int F, int E, int top,
                          void* ws, size_t ws_bytes, hipStream_t s);   // mixers_moe_mfma.hip
size_t expert_grouped_workspace(int64_t T, int K, int F, int E, int top);

}  // namespace gbxm

using namespace gbxm;

extern "C" size_t gbxm_expert_glu_workspace(int64_t T_, int32_t K, int32_t F, int32_t E, int32_t top, int32_t act) {
  return act == GBXM_BF16 ? expert_grouped_workspace(T_, K, F, E, top) : 0;
}

extern "C" int gbxm_expert_glu(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T_, int32_t K, int32_t F,
                               int32_t E, int32_t top, int32_t act, void* ws, size_t ws_bytes, void* stream) {
  if (!h || !gate_up || !down || !idx || !y || K <= 0 || F <= 0 || E <= 0 || top < 1 || top > E || T_ < 0 || (act != GBXM_BF16 && act != GBXM_F32))
    return fail(GBXM_ERR_INVALID, "expert_glu: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (act == GBXM_BF16 && ws && ws_bytes) {
    const int rc = launch_expert_grouped(h, gate_up, down, idx, y, T_, K, F, E, top, ws, ws_bytes, s);
    if (rc != GBXM_ERR_UNSUPPORTED) return rc;
  }
  const size_t lds = static_cast<size_t>(K + F) * sizeof(float);
  if (lds > 64 * 1024) return fail(GBXM_ERR_UNSUPPORTED, "expert_glu: K + F = %d beyond the row kernel's LDS", K + F);
  if (T_ * top > 0x7fffffffLL || top > 65535) return fail(GBXM_ERR_UNSUPPORTED, "expert_glu: grid");
  if (act == GBXM_BF16)
    expert_rows_kernel<bf16_t, true><<<dim3(T_ * top), NT, lds, s>>>(static_cast<const bf16_t*>(h), static_cast<const bf16_t*>(gate_up),
                                                                        static_cast<const bf16_t*>(down), idx, static_cast<bf16_t*>(y), K, F, top);
  else
    expert_rows_kernel<float, false><<<dim3(T_ * top), NT, lds, s>>>(static_cast<const float*>(h), static_cast<const float*>(gate_up),
                                                                        static_cast<const float*>(down), idx, static_cast<float*>(y), K, F, top);
  return after_launch("expert_glu");
}
