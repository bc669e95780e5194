// Gated sliding-window attention over a ragged step:  o_i = sum_{0 <= i-j < window} sigmoid(s_ij + c_h) v_j,
//   s_ij = cap * tanh(scale * <q_i, k_j> / cap) - a_h * log(1 + b_h (i - j)).
// The gates are not normalised over the keys, so there is no running maximum and no rescaling: partial sums over key tiles simply
// add.  Keys before the step's first row come from the slot's ring (row = position % window), the step's own keys from its
// projection rows -- a long portion never reads a ring row it is about to overwrite.
//
// Two kernels:
//   * window_rows_kernel  -- any head sizes, fp32 or bf16: one workgroup per (row, kv head) takes all query heads of the group,
//     scores by vector FMAs over a 64-key tile (16-byte key loads), then the value sum with the lanes across the value channels.  The
//     kernel of decode steps (one row per sequence) and of every shape the matrix-core kernel does not take; all arithmetic fp32.
//     A step of few rows splits each row's key tiles over several workgroups (fp32 partial sums, added in a fixed order by
//     window_reduce_kernel), so that one sequence's decode step still reads its window with the whole chip.
//   * window_tile_kernel  -- bf16 prompt portions on the matrix cores (second part of this file).
#include <algorithm>
#include "mixers_common.h"

namespace gbxm {
namespace {

constexpr int NT = 256;
constexpr int KT = 64;            // keys per tile of the row kernel

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

// <q, k> over dk channels: q in LDS (fp32), k a global row.  VEC: 16-byte loads (dk a multiple of the vector, row 16-byte aligned).
template <typename T, bool VEC>
__device__ __forceinline__ float qk_dot(const float* __restrict__ q, const T* __restrict__ k, int dk) {
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

constexpr int RC = 8;             // query heads a workgroup of the row kernel takes at most
constexpr int DCH = 128;          // value channels per lane pass (two per lane)
constexpr int NCH = 4;            // lane passes: value sizes up to NCH * DCH

// One workgroup = one row x one kv head x up to RC of its query heads x its share of the key tiles.
//   scores: a thread per (head, key) of a 64-key tile, 16-byte key loads against the query in LDS, gates to LDS;
//   values: a wave per key, lanes across the value channels (two each), every loaded value feeds all heads' sums;
//   the four waves' sums meet in LDS in a fixed order.
template <typename T, bool FAST, bool VEC>
__global__ __launch_bounds__(NT) void window_rows_kernel(const T* __restrict__ qkv, int64_t stride, const T* __restrict__ kc, const T* __restrict__ vc,
                                                        const int* __restrict__ seq, const int* __restrict__ tok, T* __restrict__ out,
                                                        const float* __restrict__ dmul, const float* __restrict__ drate,
                                                        const float* __restrict__ gbias, Geo g, int rc, int splits, float* __restrict__ partial) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const T** kptr = reinterpret_cast<const T**>(lds_raw);            // [KT] rows of the tile's keys
  const T** vptr = kptr + KT;                                        // [KT] and values
  float* ql = reinterpret_cast<float*>(vptr + KT);                   // [rc][dk]
  float* gl = ql + rc * g.dk;                                        // [rc][KT]
  float* sums = gl + rc * KT;                                        // [NW][rc * dv]
  constexpr int NW = NT / 64;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int R = g.H / g.G;
  const int chunks = (R + rc - 1) / rc;
  const int kvh = blockIdx.y / chunks, r0 = (blockIdx.y % chunks) * rc;
  const int nr = min(rc, R - r0);                   // query heads of this workgroup: kvh * R + r0 + (0 .. nr-1)
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], row0 = seq[4 * b + 3];
  const int nkv_k = g.G * g.dk, nkv_v = g.G * g.dv;
  const T* qrow = qkv + t * stride + (kvh * R + r0) * g.dk;
  for (int i = threadIdx.x; i < nr * g.dk; i += NT) ql[i] = to_f32(qrow[i]);
  float acc[NCH][RC][2];
#pragma unroll
  for (int c = 0; c < NCH; ++c)
#pragma unroll
    for (int r = 0; r < RC; ++r) acc[c][r][0] = acc[c][r][1] = 0.f;
  const bool pair_loads = g.dv % 2 == 0 && VEC;     // (VEC: rows are 16-byte aligned, so channel pairs are 4-byte aligned)
  const int jlo = max(0, pos - g.window + 1);
  for (int jt = jlo + static_cast<int>(blockIdx.z) * KT; jt <= pos; jt += KT * splits) {     // this workgroup's share of the key tiles
    __syncthreads();                                // the previous tile's gates and rows have been consumed
    if (threadIdx.x < KT) {
      const int j = min(jt + static_cast<int>(threadIdx.x), pos);
      kptr[threadIdx.x] = key_row(qkv, stride, kc, nkv_k, g.nq, slot, pos0, row0, g.window, j) + kvh * g.dk;
      vptr[threadIdx.x] = key_row(qkv, stride, vc, nkv_v, g.nq + g.nk, slot, pos0, row0, g.window, j) + kvh * g.dv;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nr * KT; i += NT) {
      const int r = i / KT, jj = i % KT, j = jt + jj;
      float gate = 0.f;
      if (j <= pos) {
        const float dot = qk_dot<T, VEC>(ql + r * g.dk, kptr[jj], g.dk);
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
              const float gate = gl[r * KT + jj];
              acc[c][r][0] += gate * v0;
              acc[c][r][1] += gate * v1;
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
  const int64_t hv = static_cast<int64_t>(g.H) * g.dv;
  float* prow = splits > 1 ? partial + (static_cast<int64_t>(blockIdx.z) * gridDim.x + t) * hv + (kvh * R + r0) * g.dv : nullptr;
  T* orow = out + t * hv + (kvh * R + r0) * g.dv;
  for (int i = threadIdx.x; i < nr * g.dv; i += NT) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) s += sums[w * rc * g.dv + i];
    if (prow) prow[i] = s; else orow[i] = from_f32<T>(s);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void window_reduce_kernel(const float* __restrict__ partial, T* __restrict__ out, int64_t n, int splits) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * NT + threadIdx.x;
  if (i >= n) return;
  float s4[4] = {0.f, 0.f, 0.f, 0.f};                 // four running sums (split z goes to sum z % 4): the loads of a row do not wait
  int z = 0;                                          // for each other; the order is fixed all the same
  for (; z + 4 <= splits; z += 4) {
#pragma unroll
    for (int u = 0; u < 4; ++u) s4[u] += partial[(z + u) * n + i];
  }
  for (; z < splits; ++z) s4[z & 3] += partial[z * n + i];
  out[i] = from_f32<T>((s4[0] + s4[1]) + (s4[2] + s4[3]));
}

template <typename T, bool FAST>
int launch_rows(const gbxm_window_attn_args& a, const Geo& g, int rc, int chunks, size_t lds, hipStream_t s) {
  constexpr int PER = 16 / sizeof(T);
  const bool vec = a.dk % PER == 0 && a.row_stride % PER == 0 && (a.H * a.dk) % PER == 0 &&
                   (reinterpret_cast<uintptr_t>(a.qkv) | reinterpret_cast<uintptr_t>(a.kcache)) % 16 == 0;
  // few rows: split every row's key tiles so that about two workgroups per CU exist (never more splits than tiles of a full window)
  int splits = 1;
  const int64_t groups = a.T * a.G * chunks;
  if (a.partial && groups < 256) {
    const int tiles = (a.window + KT - 1) / KT;
    splits = static_cast<int>(std::min<int64_t>(std::min<int64_t>(512 / groups, tiles), a.partial_splits));
    if (splits < 2) splits = 1;
  }
  const dim3 grid(a.T, a.G * chunks, splits);
  const T* q = static_cast<const T*>(a.qkv);
  const T* kc = static_cast<const T*>(a.kcache);
  const T* vc = static_cast<const T*>(a.vcache);
  T* out = static_cast<T*>(a.out);
  float* part = static_cast<float*>(a.partial);
  if (vec)
    window_rows_kernel<T, FAST, true><<<grid, NT, lds, s>>>(q, a.row_stride, kc, vc, a.seq, a.tok, out, a.dist_mul, a.dist_rate, a.gate_bias, g, rc, splits, part);
  else
    window_rows_kernel<T, FAST, false><<<grid, NT, lds, s>>>(q, a.row_stride, kc, vc, a.seq, a.tok, out, a.dist_mul, a.dist_rate, a.gate_bias, g, rc, splits, part);
  if (splits > 1) {
    const int64_t n = a.T * a.H * a.dv;
    window_reduce_kernel<T><<<dim3((n + NT - 1) / NT), NT, 0, s>>>(part, out, n, splits);
  }
  return after_launch("window_attention (rows)");
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
  // query heads per workgroup: at most RC, and the workgroup's LDS (rows, query, gates, the waves' sums) within 60 KB
  if (a->dv > NCH * DCH) return fail(GBXM_ERR_UNSUPPORTED, "window_attention: value size %d beyond the row kernel (%d)", a->dv, NCH * DCH);
  auto lds_of = [&](int rc_) { return static_cast<size_t>(2 * KT) * sizeof(void*) + static_cast<size_t>(rc_) * (a->dk + KT + 4 * a->dv) * sizeof(float); };
  int rc = R < RC ? R : RC;
  while (rc > 1 && lds_of(rc) > 60 * 1024) --rc;
  if (lds_of(rc) > 60 * 1024) return fail(GBXM_ERR_UNSUPPORTED, "window_attention: head sizes dk=%d dv=%d are beyond the row kernel", a->dk, a->dv);
  const int chunks = (R + rc - 1) / rc;
  const size_t lds = lds_of(rc);
  if (a->T > 0x7fffffffLL || a->G * chunks > 65535) return fail(GBXM_ERR_UNSUPPORTED, "window_attention: grid");
  return a->act == GBXM_BF16 ? launch_rows<bf16_t, true>(*a, g, rc, chunks, lds, s) : launch_rows<float, false>(*a, g, rc, chunks, lds, s);
}
