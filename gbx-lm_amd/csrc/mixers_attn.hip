// Gated sliding-window attention over a ragged step:  o_i = sum_{0 <= i-j < window} sigmoid(s_ij + c_h) v_j,
//   s_ij = cap * tanh(scale * <q_i, k_j> / cap) - a_h * log(1 + b_h (i - j)).
// The gates are not normalised over the keys, so there is no running maximum and no rescaling: partial sums over key tiles simply
// add.  Keys before the step's first row come from the slot's ring (row = position % window), the step's own keys from its
// projection rows -- a long portion never reads a ring row it is about to overwrite.
//
// Two kernels:
//   * window_rows_kernel  -- any head sizes, fp32 or bf16: one workgroup per (row, kv head) takes all query heads of the group,
//     scores by vector FMAs over a 64-key tile, then the value sum with the lanes across the value channels.  The kernel of decode
//     steps (one row per sequence) and of every shape the matrix-core kernel does not take; all arithmetic fp32.
//   * window_tile_kernel  -- bf16 prompt portions on the matrix cores (second part of this file).
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256;
constexpr int KT = 64;            // keys per tile of the row kernel
constexpr int MAXACC = 8;         // value sums a thread of the row kernel can own

struct Geo {
  int H, G, dk, dv, window, nq, nk;
  float scale, softcap;
};

template <typename T>
__device__ __forceinline__ const T* key_row(const T* qkv, int64_t stride, const T* ring, int row_elems, int seg_off, int slot, int pos0, int row0,
                                            int window, int j) {
  // position j of the sequence: ring row (before the step) or projection row (inside it); seg_off: offset of the k / v segment
  return j < pos0 ? ring + (static_cast<int64_t>(slot) * window + j % window) * row_elems
                  : qkv + (row0 + (j - pos0)) * stride + seg_off;
}

template <typename T, bool FAST>
__global__ __launch_bounds__(NT) void window_rows_kernel(const T* __restrict__ qkv, int64_t stride, const T* __restrict__ kc, const T* __restrict__ vc,
                                                        const int* __restrict__ seq, const int* __restrict__ tok, T* __restrict__ out,
                                                        const float* __restrict__ dmul, const float* __restrict__ drate,
                                                        const float* __restrict__ gbias, Geo g, int rc) {
  extern __shared__ float lds[];                    // q [rc][dk] | gates [rc][KT]
  const int64_t t = blockIdx.x;
  const int R = g.H / g.G;
  const int chunks = (R + rc - 1) / rc;
  const int kvh = blockIdx.y / chunks, r0 = (blockIdx.y % chunks) * rc;
  const int nr = min(rc, R - r0);                   // query heads of this workgroup: kvh * R + r0 + (0 .. nr-1)
  float* ql = lds;
  float* gl = lds + rc * g.dk;
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], row0 = seq[4 * b + 3];
  const int nkv_k = g.G * g.dk, nkv_v = g.G * g.dv;
  const T* qrow = qkv + t * stride + (kvh * R + r0) * g.dk;
  for (int i = threadIdx.x; i < nr * g.dk; i += NT) ql[i] = to_f32(qrow[i]);
  float acc[MAXACC];
#pragma unroll
  for (int i = 0; i < MAXACC; ++i) acc[i] = 0.f;
  const int jlo = max(0, pos - g.window + 1);
  for (int jt = jlo; jt <= pos; jt += KT) {
    __syncthreads();                                // q ready; gates of the previous tile consumed
    for (int i = threadIdx.x; i < nr * KT; i += NT) {
      const int r = i / KT, j = jt + i % KT;
      float gate = 0.f;
      if (j <= pos) {
        const T* kr = key_row(qkv, stride, kc, nkv_k, g.nq, slot, pos0, row0, g.window, j) + kvh * g.dk;
        const float* qr = ql + r * g.dk;
        float dot = 0.f;
        for (int d = 0; d < g.dk; ++d) dot += qr[d] * to_f32(kr[d]);
        const int head = kvh * R + r0 + r;
        float s = dot * g.scale;
        if (g.softcap > 0.f) s = g.softcap * tanh_<FAST>(s / g.softcap);
        s -= dmul[head] * log1p_<FAST>(drate[head] * static_cast<float>(pos - j));
        gate = sigmoid_<FAST>(s + gbias[head]);
      }
      gl[i] = gate;
    }
    __syncthreads();
    const int nj = min(KT, pos - jt + 1);
#pragma unroll
    for (int a = 0; a < MAXACC; ++a) {
      const int i = threadIdx.x + a * NT;
      if (i < nr * g.dv) {
        const int r = i / g.dv, d = i % g.dv;
        float s = acc[a];
        for (int jj = 0; jj < nj; ++jj) {
          const T* vr = key_row(qkv, stride, vc, nkv_v, g.nq + g.nk, slot, pos0, row0, g.window, jt + jj) + kvh * g.dv;
          s += gl[r * KT + jj] * to_f32(vr[d]);
        }
        acc[a] = s;
      }
    }
  }
  T* orow = out + t * (static_cast<int64_t>(g.H) * g.dv) + (kvh * R + r0) * g.dv;
#pragma unroll
  for (int a = 0; a < MAXACC; ++a) {
    const int i = threadIdx.x + a * NT;
    if (i < nr * g.dv) orow[i] = from_f32<T>(acc[a]);
  }
}

}  // namespace

int launch_window_tiles(const gbxm_window_attn_args& a, hipStream_t s);     // mixers_attn_mfma.hip; GBXM_ERR_UNSUPPORTED: not its shape
bool window_tiles_shape(int dk, int dv);

}  // namespace gbxm

using namespace gbxm;

extern "C" int gbxm_window_attention_tiled(int32_t dk, int32_t dv, int32_t act, int32_t decode_only) {
  return act == GBXM_BF16 && !decode_only && window_tiles_shape(dk, dv);
}

extern "C" int gbxm_window_attention(const gbxm_window_attn_args* a, void* stream) {
  if (!a || !a->qkv || !a->kcache || !a->vcache || !a->seq || !a->tok || !a->out || !a->dist_mul || !a->dist_rate || !a->gate_bias)
    return fail(GBXM_ERR_INVALID, "window_attention: null argument");
  if (a->act != GBXM_BF16 && a->act != GBXM_F32) return fail(GBXM_ERR_INVALID, "window_attention: dtype");
  if (a->H <= 0 || a->G <= 0 || a->H % a->G || a->dk <= 0 || a->dv <= 0 || a->window < 1 || a->T < 0 || a->B < 0)
    return fail(GBXM_ERR_INVALID, "window_attention: bad geometry");
  const int64_t need = static_cast<int64_t>(a->H) * a->dk + static_cast<int64_t>(a->G) * (a->dk + a->dv);
  if (a->row_stride < need) return fail(GBXM_ERR_INVALID, "window_attention: row stride below q|k|v");
  if (a->T == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!a->decode_only && a->act == GBXM_BF16 && a->tiles && a->n_tiles > 0) {
    const int rc = launch_window_tiles(*a, s);
    if (rc != GBXM_ERR_UNSUPPORTED) return rc;
  }
  Geo g{a->H, a->G, a->dk, a->dv, a->window, a->H * a->dk, a->G * a->dk, a->scale, a->softcap};
  const int R = a->H / a->G;
  // query heads per workgroup: bounded by the value sums its threads can own and by 48 KB of LDS
  int rc = R;
  while (rc > 1 && (static_cast<int64_t>(rc) * a->dv > MAXACC * NT || static_cast<size_t>(rc) * (a->dk + KT) * 4 > 48 * 1024)) --rc;
  if (static_cast<int64_t>(rc) * a->dv > MAXACC * NT || static_cast<size_t>(rc) * (a->dk + KT) * 4 > 48 * 1024)
    return fail(GBXM_ERR_UNSUPPORTED, "window_attention: head sizes dk=%d dv=%d are beyond the row kernel", a->dk, a->dv);
  const int chunks = (R + rc - 1) / rc;
  const size_t lds = static_cast<size_t>(rc) * (a->dk + KT) * sizeof(float);
  const dim3 grid(a->T, a->G * chunks);
  if (a->T > 0x7fffffffLL || grid.y > 65535) return fail(GBXM_ERR_UNSUPPORTED, "window_attention: grid");
  if (a->act == GBXM_BF16)
    window_rows_kernel<bf16_t, true><<<grid, NT, lds, s>>>(static_cast<const bf16_t*>(a->qkv), a->row_stride, static_cast<const bf16_t*>(a->kcache),
                                                           static_cast<const bf16_t*>(a->vcache), a->seq, a->tok, static_cast<bf16_t*>(a->out),
                                                           a->dist_mul, a->dist_rate, a->gate_bias, g, rc);
  else
    window_rows_kernel<float, false><<<grid, NT, lds, s>>>(static_cast<const float*>(a->qkv), a->row_stride, static_cast<const float*>(a->kcache),
                                                           static_cast<const float*>(a->vcache), a->seq, a->tok, static_cast<float*>(a->out),
                                                           a->dist_mul, a->dist_rate, a->gate_bias, g, rc);
  return after_launch("window_attention");
}
