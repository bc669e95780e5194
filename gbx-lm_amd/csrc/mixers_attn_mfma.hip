// Matrix-core kernel of gated sliding-window attention for bf16 prompt portions (mechanism: mixers_attn.hip).
//
// One workgroup = 4 waves = one tile of up to 128 query rows of one (sequence, head); a wave owns 32 queries.  Key / value tiles
// of 32 positions go global -> registers (one tile ahead) -> LDS once per workgroup (ring rows for positions before the step, projection rows inside it; rows
// past the tile's last query are zero-filled so that a zero gate never meets a stale NaN).  Both products are computed swapped so
// that a lane owns ONE query and the gate arithmetic is lane-local:
//   S^T[key, q] = mfma(K rows, Q rows)      lane (q = lane % 32) holds 16 keys of the tile, the other 16 are in lane ^ 32
//   O^T[d, q]  += mfma(V^T rows, G^T)       the gate operand of k-step t is the lane's own g[8t .. 8t+7]; V^T comes out of LDS by
//                                            transposed reads in the same key order
// No softmax: gates of different keys are independent, O^T just accumulates -- no running maximum, no rescale, no final division.
// The fp32 part per score (soft cap, log distance penalty, sigmoid: five transcendentals) outweighs the MFMAs: the kernel is bound
// by the quarter-rate transcendental pipe, not by the matrix cores.  Gates are rounded to bf16 for the value product.
#include "mixers_mfma.h"

namespace gbxm {
namespace {

struct TileArgs {
  const bf16_t* qkv;
  const bf16_t* kc;
  const bf16_t* vc;
  const int* seq;
  const int* tiles;
  bf16_t* out;
  const float* dmul;
  const float* drate;
  const float* gbias;
  int64_t stride;
  int q_tile, H, G, window, nq, nk;
  float scale, softcap;
};

template <int DK, int DV>
__global__ __launch_bounds__(256) void window_tile_kernel(const TileArgs a) {
  constexpr int KT = 32;
  constexpr int KROW = DK * 2 + 16;          // +16 B: conflict-free 16-byte fragment reads
  constexpr int VROW = DV * 2 + 64;          // pitch = 16 dwords mod 64: the 4 rows of a transposed block land on disjoint banks
  constexpr int KS = DK / 16, DT = DV / 32;
  __shared__ __attribute__((aligned(16))) unsigned char lds[KT * KROW + KT * VROW];
  unsigned char* kl = lds;
  unsigned char* vl = lds + KT * KROW;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, hb = lane >> 5;
  const int b = a.tiles[2 * blockIdx.x], tq = a.tiles[2 * blockIdx.x + 1];
  const int head = blockIdx.y, kvh = head / (a.H / a.G);
  const int slot = a.seq[4 * b], pos0 = a.seq[4 * b + 1], n = a.seq[4 * b + 2], row0 = a.seq[4 * b + 3];
  const int W = a.window;
  const int qn = min(a.q_tile, n - tq);                     // queries of this tile
  const int qloc = wave * 32 + r;
  const bool qvalid = qloc < qn;
  const int qpos = pos0 + tq + qloc;
  const int nkv_k = a.G * DK, nkv_v = a.G * DV;

  u32x4 qf[KS];
  {
    const bf16_t* qp = a.qkv + (row0 + tq + min(qloc, qn - 1)) * a.stride + head * DK + hb * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const u32x4*>(qp + ks * 16);
  }
  f32x16 o[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i) o[i] = f32x16{0};

  const int jfirst = max(0, pos0 + tq - W + 1), jlast = pos0 + tq + qn - 1;
  const bool wave_live = wave * 32 < qn;
  const int wq0 = pos0 + tq + wave * 32, wq1 = min(wq0 + 31, jlast);   // positions of this wave's queries
  const float dm = a.dmul[head], dr = a.drate[head], gb = a.gbias[head];
  const float cap = a.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f, scale = a.scale;
  const unsigned char* vbase = vl + (4 * hb + ((lane >> 2) & 3)) * VROW + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  const unsigned char* kbase = kl + r * KROW + hb * 16;

  auto src = [&](const bf16_t* ring, int row_elems, int seg_off, int j) -> const bf16_t* {
    return j < pos0 ? ring + (static_cast<int64_t>(slot) * W + j % W) * row_elems : a.qkv + (row0 + (j - pos0)) * a.stride + seg_off;
  };

  // key / value tile: global -> registers one tile ahead, registers -> LDS at the top of its iteration
  constexpr int KP = (KT * (DK / 8) + 255) / 256, VP = (KT * (DV / 8) + 255) / 256;
  u32x4 kr[KP], vr[VP];
  auto fetch = [&](int jt) {
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int p = tid + 256 * i, row = p / (DK / 8), c = p % (DK / 8), j = jt + row;
      kr[i] = u32x4{0, 0, 0, 0};
      if (p < KT * (DK / 8) && j <= jlast) kr[i] = *reinterpret_cast<const u32x4*>(src(a.kc, nkv_k, a.nq, j) + kvh * DK + c * 8);
    }
#pragma unroll
    for (int i = 0; i < VP; ++i) {
      const int p = tid + 256 * i, row = p / (DV / 8), c = p % (DV / 8), j = jt + row;
      vr[i] = u32x4{0, 0, 0, 0};
      if (p < KT * (DV / 8) && j <= jlast) vr[i] = *reinterpret_cast<const u32x4*>(src(a.vc, nkv_v, a.nq + a.nk, j) + kvh * DV + c * 8);
    }
  };
  fetch(jfirst);
  for (int jt = jfirst; jt <= jlast; jt += KT) {
    __syncthreads();                                          // the previous tile has been consumed
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int p = tid + 256 * i;
      if (p < KT * (DK / 8)) *reinterpret_cast<u32x4*>(kl + (p / (DK / 8)) * KROW + (p % (DK / 8)) * 16) = kr[i];
    }
#pragma unroll
    for (int i = 0; i < VP; ++i) {
      const int p = tid + 256 * i;
      if (p < KT * (DV / 8)) *reinterpret_cast<u32x4*>(vl + (p / (DV / 8)) * VROW + (p % (DV / 8)) * 16) = vr[i];
    }
    __syncthreads();
    if (jt + KT <= jlast) fetch(jt + KT);                     // the next tile travels while this one is computed
    if (!wave_live || jt > wq1 || jt + KT - 1 < wq0 - W + 1) continue;      // wave-uniform: no key of the tile is seen by this wave

    f32x16 st = f32x16{0};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) st = mfma_bf16(*reinterpret_cast<const u32x4*>(kbase + ks * 32), qf[ks], st);
    float g[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int dist = qpos - (jt + 8 * (e >> 2) + 4 * hb + (e & 3));
      float s = st[e] * scale;
      if (cap > 0.f) s = cap * tanh_<true>(s * inv_cap);
      s -= dm * __logf(1.f + dr * static_cast<float>(max(dist, 0)));
      const float v = sigmoid_<true>(s + gb);
      g[e] = (qvalid && dist >= 0 && dist < W) ? v : 0.f;
    }
    u32x4 gf[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
      gf[tt] = u32x4{pack2(g[8 * tt], g[8 * tt + 1]), pack2(g[8 * tt + 2], g[8 * tt + 3]), pack2(g[8 * tt + 4], g[8 * tt + 5]),
                     pack2(g[8 * tt + 6], g[8 * tt + 7])};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const u32x2 v0 = lds_read_tr(vbase + (16 * tt) * VROW + dt * 64);
        const u32x2 v1 = lds_read_tr(vbase + (16 * tt + 8) * VROW + dt * 64);
        o[dt] = mfma_bf16(u32x4{v0.x, v0.y, v1.x, v1.y}, gf[tt], o[dt]);
      }
  }

  if (qvalid) {
    bf16_t* op = a.out + (row0 + tq + qloc) * (static_cast<int64_t>(a.H) * DV) + head * DV;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = dt * 32 + 8 * q4 + 4 * hb;
        *reinterpret_cast<u32x2*>(op + d) = u32x2{pack2(o[dt][4 * q4], o[dt][4 * q4 + 1]), pack2(o[dt][4 * q4 + 2], o[dt][4 * q4 + 3])};
      }
  }
}

template <int DK, int DV>
int launch(const TileArgs& t, int n_tiles, int H, hipStream_t s) {
  window_tile_kernel<DK, DV><<<dim3(n_tiles, H), 256, 0, s>>>(t);
  return after_launch("window_attention (tiles)");
}

}  // namespace

bool window_tiles_shape(int dk, int dv) {
  const int ok[][2] = {{64, 64}, {96, 64}, {128, 64}, {64, 128}, {128, 128}, {192, 128}, {256, 256}, {96, 96}, {64, 32}, {32, 32}, {32, 64}};
  for (const auto& p : ok)
    if (p[0] == dk && p[1] == dv) return true;
  return false;
}

int launch_window_tiles(const gbxm_window_attn_args& a, hipStream_t s) {
  if (!window_tiles_shape(a.dk, a.dv)) return GBXM_ERR_UNSUPPORTED;
  if (a.q_tile != 128 || a.H > 65535 || a.row_stride % 8 || (reinterpret_cast<uintptr_t>(a.qkv) | reinterpret_cast<uintptr_t>(a.kcache) |
                                                             reinterpret_cast<uintptr_t>(a.vcache) | reinterpret_cast<uintptr_t>(a.out)) % 16)
    return GBXM_ERR_UNSUPPORTED;
  TileArgs t{static_cast<const bf16_t*>(a.qkv), static_cast<const bf16_t*>(a.kcache), static_cast<const bf16_t*>(a.vcache), a.seq, a.tiles,
             static_cast<bf16_t*>(a.out), a.dist_mul, a.dist_rate, a.gate_bias, a.row_stride, a.q_tile, a.H, a.G, a.window, a.H * a.dk,
             a.G * a.dk, a.scale, a.softcap};
#define GBXM_TILE(DK_, DV_) if (a.dk == DK_ && a.dv == DV_) return launch<DK_, DV_>(t, a.n_tiles, a.H, s)
  GBXM_TILE(64, 64); GBXM_TILE(96, 64); GBXM_TILE(128, 64); GBXM_TILE(64, 128); GBXM_TILE(128, 128); GBXM_TILE(192, 128); GBXM_TILE(256, 256);
  GBXM_TILE(96, 96); GBXM_TILE(64, 32); GBXM_TILE(32, 32); GBXM_TILE(32, 64);
#undef GBXM_TILE
  return GBXM_ERR_UNSUPPORTED;
}

}  // namespace gbxm
