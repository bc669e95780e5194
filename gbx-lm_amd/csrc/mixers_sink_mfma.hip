// Matrix-core kernel of softmax attention with a sink for bf16 prompt portions (mechanism and key order: mixers_sink.hip).
//
// One workgroup = 4 waves = one tile of up to 128 query rows of one (sequence, head); a wave owns 32 queries.  Key / value tiles
// of 32 visible positions go global -> registers (one tile ahead) -> LDS once per workgroup.  Both products are computed swapped,
//   S^T[key, q] = mfma(K rows, Q rows),    O^T[d, q] += mfma(V^T rows, P^T),
// so that a lane owns ONE query: lane (q = lane % 32, half = lane / 32) holds 16 of the tile's 32 scores of its query, the other 16
// are in lane ^ 32.  The running maximum is shared by the two lanes of a query (one cross-lane exchange per tile), each keeps its
// own part of the denominator (joined once at the end), and both rescale their accumulators (different channels of the same
// query) by the same factor.  The sink starts the running maximum and counts once in the denominator.  Weights are rounded to bf16
// for the value product; the denominator sums them in fp32.
//
// Head sizes are run-time numbers (multiples of 8) inside a compiled capacity <DK, DV>: channels beyond them are staged as zeros.
#include <algorithm>
#include "mixers_mfma.h"

namespace gbxm {

int launch_sink_reduce(const gbxm_sink_attn_args& a, int splits, hipStream_t s);      // mixers_sink.hip

namespace {

struct SinkTileArgs {
  const bf16_t* q;
  const bf16_t* kn;
  const bf16_t* vn;
  const bf16_t* kc;
  const bf16_t* vc;
  const int* seq;
  const int* tiles;
  bf16_t* out;
  const float* sink;
  const bf16_t* gate;
  int64_t q_row, q_head, k_row, k_head, v_row, v_head, kc_slot, kc_row, kc_head, vc_slot, vc_row, vc_head, gate_row;
  int q_tile, H, G, dk, dv, window, keep, ring;
  float scale;
};

template <int DK, int DV>
__device__ __forceinline__ void sink_tile(const SinkTileArgs& a, const int tile, unsigned char* lds) {
  constexpr int KT = 32;
  constexpr int KROW = DK * 2 + 16;          // +16 B: conflict-free 16-byte fragment reads
  constexpr int VROW = DV * 2 + 64;          // pitch = 16 dwords mod 64: the 4 rows of a transposed block land on disjoint banks
  constexpr int KS = DK / 16, DT = DV / 32;
  unsigned char* kl = lds;
  unsigned char* vl = lds + KT * KROW;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, hb = lane >> 5;
  const int b = a.tiles[2 * tile], tq = a.tiles[2 * tile + 1];
  const int head = blockIdx.y, kvh = head / (a.H / a.G);
  const int slot = a.seq[4 * b], pos0 = a.seq[4 * b + 1], n = a.seq[4 * b + 2], row0 = a.seq[4 * b + 3];
  const int W = a.window;
  const int qn = min(a.q_tile, n - tq);                     // queries of this tile
  const int qloc = wave * 32 + r;
  const bool qvalid = qloc < qn;
  const int qpos = pos0 + tq + qloc;

  u32x4 qf[KS];
  {
    const bf16_t* qp = a.q + (row0 + tq + min(qloc, qn - 1)) * a.q_row + head * a.q_head;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c = ks * 16 + hb * 8;
      qf[ks] = c < a.dk ? *reinterpret_cast<const u32x4*>(qp + c) : u32x4{0, 0, 0, 0};
    }
  }
  f32x16 o[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i) o[i] = f32x16{0};

  // the keys any query of the tile sees, as one run of indices: [0, na) are positions 0 .. na-1, the rest lo .. jlast
  const int qfirst = pos0 + tq, jlast = qfirst + qn - 1;
  const int lo = W > 0 ? max(0, qfirst - W + 1) : 0;
  const int na = min(a.keep, lo);
  const int total = na + (jlast - lo + 1);
  auto pos_of = [&](int iv) { return iv < na ? iv : lo + (iv - na); };
  const bool wave_live = wave * 32 < qn;
  const int wq0 = qfirst + wave * 32, wq1 = min(wq0 + 31, jlast);      // positions of this wave's queries

  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = a.scale * LOG2E;
  float m = a.sink ? a.sink[head] * LOG2E : -INFINITY;
  float l = (a.sink && hb == 0) ? 1.f : 0.f;                            // the sink counts once per query
  const unsigned char* vbase = vl + (4 * hb + ((lane >> 2) & 3)) * VROW + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  const unsigned char* kbase = kl + r * KROW + hb * 16;

  auto krow = [&](int j) -> const bf16_t* {
    if (j < pos0) return a.kc + slot * a.kc_slot + static_cast<int64_t>(j < a.keep ? j : a.keep + (j - a.keep) % a.ring) * a.kc_row + kvh * a.kc_head;
    return a.kn + static_cast<int64_t>(row0 + (j - pos0)) * a.k_row + kvh * a.k_head;
  };
  auto vrow = [&](int j) -> const bf16_t* {
    if (j < pos0) return a.vc + slot * a.vc_slot + static_cast<int64_t>(j < a.keep ? j : a.keep + (j - a.keep) % a.ring) * a.vc_row + kvh * a.vc_head;
    return a.vn + static_cast<int64_t>(row0 + (j - pos0)) * a.v_row + kvh * a.v_head;
  };

  constexpr int KP = (KT * (DK / 8) + 255) / 256, VP = (KT * (DV / 8) + 255) / 256;
  u32x4 kr[KP], vr[VP];
  auto fetch = [&](int it) {
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int p = tid + 256 * i, row = p / (DK / 8), c = p % (DK / 8), iv = it + row;
      kr[i] = u32x4{0, 0, 0, 0};
      if (p < KT * (DK / 8) && iv < total && c * 8 < a.dk) kr[i] = *reinterpret_cast<const u32x4*>(krow(pos_of(iv)) + c * 8);
    }
#pragma unroll
    for (int i = 0; i < VP; ++i) {
      const int p = tid + 256 * i, row = p / (DV / 8), c = p % (DV / 8), iv = it + row;
      vr[i] = u32x4{0, 0, 0, 0};
      if (p < KT * (DV / 8) && iv < total && c * 8 < a.dv) vr[i] = *reinterpret_cast<const u32x4*>(vrow(pos_of(iv)) + c * 8);
    }
  };
  fetch(0);
  for (int it = 0; it < total; it += KT) {
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
    if (it + KT < total) fetch(it + KT);                      // the next tile travels while this one is computed
    // wave-uniform: no key of the tile is seen by a query of this wave
    const int jmin = pos_of(it), jmax = pos_of(min(it + KT, total) - 1);
    if (!wave_live || jmin > wq1 || (W > 0 && jmax < wq0 - W + 1 && jmin >= a.keep)) continue;

    f32x16 st = f32x16{0};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) st = mfma_bf16(*reinterpret_cast<const u32x4*>(kbase + ks * 32), qf[ks], st);
    // scores in units of ln 2 (the exponentials below are base 2).  Inside the mask -- every key of the tile before every query of the
    // wave, inside every window -- nothing is tested per score.
    const bool inside = it + KT <= total && jmax <= wq0 && (W <= 0 || wq1 - jmin < W || jmax < a.keep);
    float s[16];
    float mx = -INFINITY;
    if (inside) {
#pragma unroll
      for (int e = 0; e < 16; ++e) { s[e] = st[e] * scale2; mx = fmaxf(mx, s[e]); }
    } else {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int iv = it + 8 * (e >> 2) + 4 * hb + (e & 3);
        const int j = pos_of(iv);
        const bool seen = qvalid && iv < total && j <= qpos && (W <= 0 || qpos - j < W || j < a.keep);
        s[e] = seen ? st[e] * scale2 : -INFINITY;
        mx = fmaxf(mx, s[e]);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));                   // the other half of the query's scores
    const float m_new = fmaxf(m, mx);
    const float m_ref = m_new == -INFINITY ? 0.f : m_new;     // nothing seen yet and no sink: every weight below is 2^-inf = 0
    const float alpha = __builtin_amdgcn_exp2f(m - m_ref);
    const bool moved = m_new != m;
    m = m_new;
    float ps = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) { s[e] = __builtin_amdgcn_exp2f(s[e] - m_ref); ps += s[e]; }
    l = l * alpha + ps;
    if (__any(moved)) {                                       // wave-uniform: the maximum of no query of the wave has moved -> alpha is 1
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[dt][e] *= alpha;
    }
    u32x4 gf[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
      gf[tt] = u32x4{pack2(s[8 * tt], s[8 * tt + 1]), pack2(s[8 * tt + 2], s[8 * tt + 3]), pack2(s[8 * tt + 4], s[8 * tt + 5]),
                     pack2(s[8 * tt + 6], s[8 * tt + 7])};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const u32x2 v0 = lds_read_tr(vbase + (16 * tt) * VROW + dt * 64);
        const u32x2 v1 = lds_read_tr(vbase + (16 * tt + 8) * VROW + dt * 64);
        o[dt] = mfma_bf16(u32x4{v0.x, v0.y, v1.x, v1.y}, gf[tt], o[dt]);
      }
  }

  l += __shfl_xor(l, 32, 64);
  if (qvalid) {
    const int64_t row = row0 + tq + qloc;
    float f = 1.f / l;
    if (a.gate) f *= sigmoid_<true>(to_f32(a.gate[row * a.gate_row + head]));
    bf16_t* op = a.out + row * (static_cast<int64_t>(a.H) * a.dv) + head * a.dv;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = dt * 32 + 8 * q4 + 4 * hb;
        if (d < a.dv)                                          // dv is a multiple of 8: the four channels are inside together
          *reinterpret_cast<u32x2*>(op + d) = u32x2{pack2(o[dt][4 * q4] * f, o[dt][4 * q4 + 1] * f), pack2(o[dt][4 * q4 + 2] * f, o[dt][4 * q4 + 3] * f)};
      }
  }
}

// Steps of single rows (decoding): the query heads that share a key/value head are the 32 "query rows" of the same two products,
// all at one position, so a key tile staged once serves every head of the group.  One workgroup = one (row, kv head, 32 heads of
// its group, share of the key tiles); every wave forms all scores of a tile (the weights must be the same in all of them) and
// owns every fourth 32-channel block of the value product.  No mask besides the end of the key run.  With key splits a workgroup
// leaves (sum, maximum, denominator) per head for sink_reduce_kernel, else it finishes the row itself.
// ALIAS: the values are the first dv channels of the key rows (one staged tile serves both products).
template <int DK, int DV, bool ALIAS>
__global__ __launch_bounds__(256) void sink_group_kernel(const SinkTileArgs a, const int* __restrict__ tok, int splits, float* __restrict__ partial) {
  constexpr int KT = 32;
  constexpr int KROW = DK * 2 + 16;
  constexpr int VROW = ALIAS ? KROW : DV * 2 + 64;
  constexpr int KS = DK / 16, DT = DV / 32, DTW = (DT + 3) / 4;
  // long rows: the channels of the score product are shared out over the four waves (a quarter of the dependent matrix-core steps
  // and of the query fragments each); the four partial score tiles meet in LDS and every wave adds them in the same order, so all
  // waves hold identical scores.  The registers this frees hold the next key tile while the current one is computed.
  constexpr bool SPLITK = KS >= 16;
  constexpr int KSW = SPLITK ? (KS + 3) / 4 : KS;
  constexpr int TILE_BYTES = KT * KROW + (ALIAS ? 0 : KT * VROW);
  __shared__ __attribute__((aligned(16))) unsigned char lds[TILE_BYTES + (SPLITK ? 4 * 16 * 64 * 4 : 0)];
  unsigned char* kl = lds;
  unsigned char* vl = ALIAS ? lds : lds + KT * KROW;
  float* sred = reinterpret_cast<float*>(lds + TILE_BYTES);            // [4 waves][16][64 lanes]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, hb = lane >> 5;
  const int64_t t = blockIdx.x;
  const int R = a.H / a.G, chunks = (R + 31) / 32;
  const int kvh = blockIdx.y / chunks, hloc = (blockIdx.y % chunks) * 32 + r;
  const bool hvalid = hloc < R;
  const int head = kvh * R + min(hloc, R - 1);
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = a.seq[4 * b], pos0 = a.seq[4 * b + 1], row0 = a.seq[4 * b + 3];
  const int W = a.window;

  const int ks0 = SPLITK ? wave * KSW : 0;                              // this wave's steps of the score product: ks0 .. ks0 + KSW - 1
  u32x4 qf[KSW];
  {
    const bf16_t* qp = a.q + t * a.q_row + head * a.q_head;
#pragma unroll
    for (int i = 0; i < KSW; ++i) {
      const int c = (ks0 + i) * 16 + hb * 8;
      qf[i] = (ks0 + i < KS && c < a.dk) ? *reinterpret_cast<const u32x4*>(qp + c) : u32x4{0, 0, 0, 0};
    }
  }
  f32x16 o[DTW];
#pragma unroll
  for (int i = 0; i < DTW; ++i) o[i] = f32x16{0};

  const int lo = W > 0 ? max(0, pos - W + 1) : 0;
  const int na = min(a.keep, lo);
  const int total = na + (pos - lo + 1);
  auto pos_of = [&](int iv) { return iv < na ? iv : lo + (iv - na); };
  auto krow = [&](int j) -> const bf16_t* {
    if (j < pos0) return a.kc + slot * a.kc_slot + static_cast<int64_t>(j < a.keep ? j : a.keep + (j - a.keep) % a.ring) * a.kc_row + kvh * a.kc_head;
    return a.kn + static_cast<int64_t>(row0 + (j - pos0)) * a.k_row + kvh * a.k_head;
  };
  auto vrow = [&](int j) -> const bf16_t* {
    if (j < pos0) return a.vc + slot * a.vc_slot + static_cast<int64_t>(j < a.keep ? j : a.keep + (j - a.keep) % a.ring) * a.vc_row + kvh * a.vc_head;
    return a.vn + static_cast<int64_t>(row0 + (j - pos0)) * a.v_row + kvh * a.v_head;
  };

  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = a.scale * LOG2E;
  const bool own_sink = a.sink && splits == 1;                          // split key tiles: the sink joins in the reduce
  float m = own_sink ? a.sink[head] * LOG2E : -INFINITY;
  float l = (own_sink && hb == 0) ? 1.f : 0.f;
  const unsigned char* vbase = vl + (4 * hb + ((lane >> 2) & 3)) * VROW + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  const unsigned char* kbase = kl + r * KROW + hb * 16;

  // a key (and value) tile: global -> registers -> LDS; with SPLITK the registers are filled one tile ahead
  constexpr int KP = (KT * (DK / 8) + 255) / 256, VP = ALIAS ? 1 : (KT * (DV / 8) + 255) / 256;
  u32x4 kr[KP], vr[VP];
  auto fetch = [&](int it) {
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int p = tid + 256 * i, row = p / (DK / 8), c = p % (DK / 8), iv = it + row;
      kr[i] = u32x4{0, 0, 0, 0};
      if (p < KT * (DK / 8) && iv < total && c * 8 < a.dk) kr[i] = *reinterpret_cast<const u32x4*>(krow(pos_of(iv)) + c * 8);
    }
    if constexpr (!ALIAS) {
#pragma unroll
      for (int i = 0; i < VP; ++i) {
        const int p = tid + 256 * i, row = p / (DV / 8), c = p % (DV / 8), iv = it + row;
        vr[i] = u32x4{0, 0, 0, 0};
        if (p < KT * (DV / 8) && iv < total && c * 8 < a.dv) vr[i] = *reinterpret_cast<const u32x4*>(vrow(pos_of(iv)) + c * 8);
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int p = tid + 256 * i;
      if (p < KT * (DK / 8)) *reinterpret_cast<u32x4*>(kl + (p / (DK / 8)) * KROW + (p % (DK / 8)) * 16) = kr[i];
    }
    if constexpr (!ALIAS) {
#pragma unroll
      for (int i = 0; i < VP; ++i) {
        const int p = tid + 256 * i;
        if (p < KT * (DV / 8)) *reinterpret_cast<u32x4*>(vl + (p / (DV / 8)) * VROW + (p % (DV / 8)) * 16) = vr[i];
      }
    }
  };

  const int it0 = static_cast<int>(blockIdx.z) * KT, step = KT * splits;
  if (SPLITK && it0 < total) fetch(it0);
  for (int it = it0; it < total; it += step) {
    if constexpr (!SPLITK) fetch(it);
    __syncthreads();                                          // the previous tile (and its partial scores) have been consumed
    stage();
    __syncthreads();
    if (SPLITK && it + step < total) fetch(it + step);        // the next tile travels while this one is computed
    f32x16 st = f32x16{0};
#pragma unroll
    for (int i = 0; i < KSW; ++i)
      if (ks0 + i < KS) st = mfma_bf16(*reinterpret_cast<const u32x4*>(kbase + (ks0 + i) * 32), qf[i], st);      // wave-uniform test
    if constexpr (SPLITK) {
#pragma unroll
      for (int e = 0; e < 16; ++e) sred[(wave * 16 + e) * 64 + lane] = st[e];
      __syncthreads();
#pragma unroll
      for (int e = 0; e < 16; ++e)
        st[e] = (sred[e * 64 + lane] + sred[(16 + e) * 64 + lane]) + (sred[(32 + e) * 64 + lane] + sred[(48 + e) * 64 + lane]);
    }
    float s[16];
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int iv = it + 8 * (e >> 2) + 4 * hb + (e & 3);
      s[e] = iv < total ? st[e] * scale2 : -INFINITY;
      mx = fmaxf(mx, s[e]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));                   // finite: a tile holds at least one key
    const float m_new = fmaxf(m, mx);
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    m = m_new;
    float ps = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) { s[e] = __builtin_amdgcn_exp2f(s[e] - m_new); ps += s[e]; }
    l = l * alpha + ps;
    u32x4 gf[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
      gf[tt] = u32x4{pack2(s[8 * tt], s[8 * tt + 1]), pack2(s[8 * tt + 2], s[8 * tt + 3]), pack2(s[8 * tt + 4], s[8 * tt + 5]),
                     pack2(s[8 * tt + 6], s[8 * tt + 7])};
#pragma unroll
    for (int i = 0; i < DTW; ++i) {
      const int dt = wave + 4 * i;                            // wave-uniform
      if (dt < DT) {
#pragma unroll
        for (int e = 0; e < 16; ++e) o[i][e] *= alpha;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
          const u32x2 v0 = lds_read_tr(vbase + (16 * tt) * VROW + dt * 64);
          const u32x2 v1 = lds_read_tr(vbase + (16 * tt + 8) * VROW + dt * 64);
          o[i] = mfma_bf16(u32x4{v0.x, v0.y, v1.x, v1.y}, gf[tt], o[i]);
        }
      }
    }
  }

  l += __shfl_xor(l, 32, 64);
  if (!hvalid) return;
  if (splits > 1) {
    const int pw = partial_width(a.dv);
    float* prow = partial + ((static_cast<int64_t>(blockIdx.z) * gridDim.x + t) * a.H + head) * pw;
#pragma unroll
    for (int i = 0; i < DTW; ++i) {
      const int dt = wave + 4 * i;
      if (dt < DT)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int d = dt * 32 + 8 * q4 + 4 * hb;
          if (d < a.dv) *reinterpret_cast<float4*>(prow + d) = float4{o[i][4 * q4], o[i][4 * q4 + 1], o[i][4 * q4 + 2], o[i][4 * q4 + 3]};
        }
    }
    if (wave == 0 && hb == 0) { prow[pw - 2] = m / LOG2E; prow[pw - 1] = l; }
    return;
  }
  float f = 1.f / l;
  if (a.gate) f *= sigmoid_<true>(to_f32(a.gate[t * a.gate_row + head]));
  bf16_t* op = a.out + t * (static_cast<int64_t>(a.H) * a.dv) + head * a.dv;
#pragma unroll
  for (int i = 0; i < DTW; ++i) {
    const int dt = wave + 4 * i;
    if (dt < DT)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = dt * 32 + 8 * q4 + 4 * hb;
        if (d < a.dv)
          *reinterpret_cast<u32x2*>(op + d) = u32x2{pack2(o[i][4 * q4] * f, o[i][4 * q4 + 1] * f), pack2(o[i][4 * q4 + 2] * f, o[i][4 * q4 + 3] * f)};
      }
  }
}

template <int DK, int DV, bool ALIAS>
int launch_group(const SinkTileArgs& t, const gbxm_sink_attn_args& a, hipStream_t s) {
  const int R = a.H / a.G, chunks = (R + 31) / 32;
  int splits = 1;
  const int64_t groups = a.T * a.G * chunks;
  if (a.partial && a.partial_splits > 1 && groups < 256) {
    splits = static_cast<int>(std::min<int64_t>(std::min<int64_t>(512 / groups, 64), a.partial_splits));
    if (splits < 2) splits = 1;
  }
  sink_group_kernel<DK, DV, ALIAS><<<dim3(a.T, a.G * chunks, splits), 256, 0, s>>>(t, a.tok, splits, static_cast<float*>(a.partial));
  const int rc = after_launch("sink_attention (grouped rows)");
  if (rc != GBXM_OK || splits == 1) return rc;
  return launch_sink_reduce(a, splits, s);
}

// A workgroup takes two query tiles, one from each end of the step's list: in a long causal prompt a late tile (many keys) and an
// early one (few), so that workgroups carry about the same work however they are spread over the chip.
template <int DK, int DV>
__global__ __launch_bounds__(256, (DK + DV <= 320 ? 2 : 1)) void sink_tile_kernel(const SinkTileArgs a, const int n_tiles) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[32 * (DK * 2 + 16) + 32 * (DV * 2 + 64)];
  const int first = n_tiles - 1 - blockIdx.x, second = blockIdx.x;
  sink_tile<DK, DV>(a, first, lds);
  if (second != first) sink_tile<DK, DV>(a, second, lds);
}

template <int DK, int DV>
int launch(const SinkTileArgs& t, int n_tiles, hipStream_t s) {
  sink_tile_kernel<DK, DV><<<dim3((n_tiles + 1) / 2, t.H), 256, 0, s>>>(t, n_tiles);
  return after_launch("sink_attention (tiles)");
}

constexpr int CAPS[][2] = {{32, 32}, {64, 64}, {64, 128}, {96, 96}, {128, 128}, {192, 128}, {256, 256}};

}  // namespace

bool sink_tiles_shape(int dk, int dv) {
  if (dk % 8 || dv % 8) return false;
  for (const auto& c : CAPS)
    if (dk <= c[0] && dv <= c[1]) return true;
  return false;
}

static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

static bool tile_operands(const gbxm_sink_attn_args& a) {
  if ((a.q_row | a.q_head | a.k_row | a.k_head | a.v_row | a.v_head) % 8 || !aligned16(a.q) || !aligned16(a.k_new) || !aligned16(a.v_new) ||
      !aligned16(a.out))
    return false;
  if (a.kcache && ((a.kc_slot | a.kc_row | a.kc_head | a.vc_slot | a.vc_row | a.vc_head) % 8 || !aligned16(a.kcache) || !aligned16(a.vcache))) return false;
  return true;
}

static SinkTileArgs tile_args(const gbxm_sink_attn_args& a) {
  return SinkTileArgs{static_cast<const bf16_t*>(a.q), static_cast<const bf16_t*>(a.k_new), static_cast<const bf16_t*>(a.v_new),
                      static_cast<const bf16_t*>(a.kcache), static_cast<const bf16_t*>(a.vcache), a.seq, a.tiles, static_cast<bf16_t*>(a.out), a.sink,
                      static_cast<const bf16_t*>(a.gate), a.q_row, a.q_head, a.k_row, a.k_head, a.v_row, a.v_head, a.kc_slot, a.kc_row, a.kc_head,
                      a.vc_slot, a.vc_row, a.vc_head, a.gate_row, a.q_tile, a.H, a.G, a.dk, a.dv, a.window, a.keep, a.ring, a.scale};
}

int launch_sink_tiles(const gbxm_sink_attn_args& a, hipStream_t s) {
  if (!sink_tiles_shape(a.dk, a.dv) || a.q_tile != 128 || a.H > 65535 || !tile_operands(a)) return GBXM_ERR_UNSUPPORTED;
  const SinkTileArgs t = tile_args(a);
#define GBXM_TILE(DK_, DV_) if (a.dk <= DK_ && a.dv <= DV_) return launch<DK_, DV_>(t, a.n_tiles, s)
  GBXM_TILE(32, 32); GBXM_TILE(64, 64); GBXM_TILE(64, 128); GBXM_TILE(96, 96); GBXM_TILE(128, 128); GBXM_TILE(192, 128); GBXM_TILE(256, 256);
#undef GBXM_TILE
  return GBXM_ERR_UNSUPPORTED;
}

// values that are the leading channels of the key rows (same buffers, same strides): one staged tile serves both products
static bool values_alias_keys(const gbxm_sink_attn_args& a) {
  return a.G == 1 && a.dv <= a.dk && a.v_new == a.k_new && (a.T == 1 || a.v_row == a.k_row) &&     // (one row: its stride is never used)
         (!a.kcache || (a.vcache == a.kcache && a.vc_slot == a.kc_slot && a.vc_row == a.kc_row));
}

bool sink_group_shape(int dk, int dv, bool alias) {
  if (dk % 8 || dv % 8) return false;
  if (alias) return dk <= 576 && dv <= 512;
  return sink_tiles_shape(dk, dv);
}

int launch_sink_group(const gbxm_sink_attn_args& a, hipStream_t s) {
  const bool alias = values_alias_keys(a);
  const int chunks = (a.H / a.G + 31) / 32;
  if (!sink_group_shape(a.dk, a.dv, alias) || a.G * chunks > 65535 || !tile_operands(a)) return GBXM_ERR_UNSUPPORTED;
  const SinkTileArgs t = tile_args(a);
  if (alias) {
#define GBXM_GROUP(DK_, DV_) if (a.dk <= DK_ && a.dv <= DV_) return launch_group<DK_, DV_, true>(t, a, s)
    GBXM_GROUP(96, 96); GBXM_GROUP(160, 128); GBXM_GROUP(320, 256); GBXM_GROUP(576, 512);
#undef GBXM_GROUP
    return GBXM_ERR_UNSUPPORTED;
  }
#define GBXM_GROUP(DK_, DV_) if (a.dk <= DK_ && a.dv <= DV_) return launch_group<DK_, DV_, false>(t, a, s)
  GBXM_GROUP(32, 32); GBXM_GROUP(64, 64); GBXM_GROUP(64, 128); GBXM_GROUP(96, 96); GBXM_GROUP(128, 128); GBXM_GROUP(192, 128); GBXM_GROUP(256, 256);
#undef GBXM_GROUP
  return GBXM_ERR_UNSUPPORTED;
}

}  // namespace gbxm
