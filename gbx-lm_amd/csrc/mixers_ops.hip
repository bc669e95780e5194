// Row kernels of ragged steps: embedding, segment norms, the branch-norm residual update, the last norm, the router and the
// append to the window rings.  One workgroup per row; statistics in fp32 with a fixed summation order, so a row's result does
// not depend on which other rows share the step.
#include "mixers_common.h"

namespace gbxm {

thread_local char g_err[512] = "";
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
int hip_fail(hipError_t e, const char* what) { return fail(GBXM_ERR_HIP, "%s: %s", what, hipGetErrorString(e)); }

namespace {

constexpr int NT = 256, NW = NT / 64;

template <typename T>
__global__ __launch_bounds__(NT) void embed_kernel(const T* __restrict__ table, const int64_t* __restrict__ tokens, float* __restrict__ x,
                                                   T* __restrict__ h, int width, float scale) {
  const int64_t t = blockIdx.x;
  const T* row = table + tokens[t] * width;
  for (int c = threadIdx.x; c < width; c += NT) {
    const float v = to_f32(row[c]) * scale;
    x[t * width + c] = v;
    if (h) h[t * width + c] = from_f32<T>(v);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void segment_rmsnorm_kernel(T* __restrict__ rows, int64_t stride, int n0, int n1, const float* __restrict__ w0,
                                                            const float* __restrict__ w1, float eps) {
  constexpr int VR = 16;                   // values a thread keeps between the two passes
  __shared__ float red[NW];
  const int seg = blockIdx.y;
  T* p = rows + blockIdx.x * stride + (seg ? n0 : 0);
  const int n = seg ? n1 : n0;
  const float* w = seg ? w1 : w0;
  float vr[VR];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VR; ++i) {
    const int c = threadIdx.x + i * NT;
    vr[i] = c < n ? to_f32(p[c]) : 0.f;
    ss += vr[i] * vr[i];
  }
  for (int c = threadIdx.x + VR * NT; c < n; c += NT) { const float v = to_f32(p[c]); ss += v * v; }
  ss = block_sum<NW>(ss, red);
  const float r = 1.f / sqrtf(ss / n + eps);
#pragma unroll
  for (int i = 0; i < VR; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < n) p[c] = from_f32<T>(vr[i] * r * w[c]);
  }
  for (int c = threadIdx.x + VR * NT; c < n; c += NT) p[c] = from_f32<T>(to_f32(p[c]) * r * w[c]);
}

constexpr int ZR = 16;             // branch values a thread keeps between the statistic and the update (rows up to ZR * NT wide)

template <typename T>
__global__ __launch_bounds__(NT) void residual_norm_add_kernel(float* __restrict__ x, const T* __restrict__ branch, const float* __restrict__ mix,
                                                              const float* __restrict__ w, T* __restrict__ h, int width, int top, float eps,
                                                              float mult) {
  __shared__ float red[NW];
  __shared__ float ml[64];
  const int64_t t = blockIdx.x;
  const T* b = branch + t * top * width;
  const bool mixed = mix != nullptr;
  if (mixed && threadIdx.x < min(top, 64)) ml[threadIdx.x] = mix[t * top + threadIdx.x];
  __syncthreads();
  auto z_at = [&](int c) {
    if (!mixed) return to_f32(b[c]);
    float z = 0.f;
    for (int s = 0; s < top; ++s) z += (s < 64 ? ml[s] : mix[t * top + s]) * to_f32(b[s * width + c]);
    return z;
  };
  float zr[ZR];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < ZR; ++i) {
    const int c = threadIdx.x + i * NT;
    zr[i] = c < width ? z_at(c) : 0.f;
    ss += zr[i] * zr[i];
  }
  for (int c = threadIdx.x + ZR * NT; c < width; c += NT) { const float z = z_at(c); ss += z * z; }
  ss = block_sum<NW>(ss, red);
  const float r = 1.f / sqrtf(ss / width + eps);
#pragma unroll
  for (int i = 0; i < ZR; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < width) {
      const float v = x[t * width + c] + mult * (zr[i] * r * w[c]);
      x[t * width + c] = v;
      if (h) h[t * width + c] = from_f32<T>(v);
    }
  }
  for (int c = threadIdx.x + ZR * NT; c < width; c += NT) {
    const float v = x[t * width + c] + mult * (z_at(c) * r * w[c]);
    x[t * width + c] = v;
    if (h) h[t * width + c] = from_f32<T>(v);
  }
}

template <typename T>
__global__ __launch_bounds__(NT) void stream_rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w, T* __restrict__ out, int width,
                                                           float eps) {
  __shared__ float red[NW];
  const int64_t t = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += NT) { const float v = x[t * width + c]; ss += v * v; }
  ss = block_sum<NW>(ss, red);
  const float r = 1.f / sqrtf(ss / width + eps);
  for (int c = threadIdx.x; c < width; c += NT) out[t * width + c] = from_f32<T>(x[t * width + c] * r * w[c]);
}

// Softmax over all experts and `top` rounds of arg-max on a row of fp32 router logits (the logits are a plain fp32 matrix product:
// the vendor library's); one workgroup per row.
__global__ __launch_bounds__(NT) void route_topk_kernel(const float* __restrict__ logits, int* __restrict__ idx, float* __restrict__ weight, int E,
                                                       int top, int renorm) {
  extern __shared__ float lg[];            // [E] logits, then probabilities
  __shared__ float red[NW];
  __shared__ float bestv[NW];
  __shared__ int besti[NW];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int e = threadIdx.x; e < E; e += NT) lg[e] = logits[t * E + e];
  __syncthreads();
  float mx = -INFINITY;
  for (int e = threadIdx.x; e < E; e += NT) mx = fmaxf(mx, lg[e]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = red[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) mx = fmaxf(mx, red[i]);
  float sum = 0.f;
  for (int e = threadIdx.x; e < E; e += NT) { const float p = expf(lg[e] - mx); lg[e] = p; sum += p; }
  sum = block_sum<NW>(sum, red);
  for (int e = threadIdx.x; e < E; e += NT) lg[e] = lg[e] / sum;
  __syncthreads();
  float chosen_sum = 0.f;
  for (int s = 0; s < top; ++s) {
    float bv = -1.f;
    int bi = 0x7fffffff;
    for (int e = threadIdx.x; e < E; e += NT)
      if (lg[e] > bv) { bv = lg[e]; bi = e; }                  // ascending e per thread: the first of equals stays
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (lane == 0) { bestv[wave] = bv; besti[wave] = bi; }
    __syncthreads();
    bv = bestv[0]; bi = besti[0];
#pragma unroll
    for (int i = 1; i < NW; ++i)
      if (bestv[i] > bv || (bestv[i] == bv && besti[i] < bi)) { bv = bestv[i]; bi = besti[i]; }
    __syncthreads();
    if (threadIdx.x == 0) { idx[t * top + s] = bi; weight[t * top + s] = bv; lg[bi] = -2.f; }
    chosen_sum += bv;
    __syncthreads();
  }
  if (renorm && threadIdx.x < top) weight[t * top + threadIdx.x] /= chosen_sum;
}

template <typename T>
__global__ __launch_bounds__(NT) void window_append_kernel(const T* __restrict__ qkv, int64_t stride, int nq, int nk, int nv, T* __restrict__ kc,
                                                          T* __restrict__ vc, const int* __restrict__ seq, const int* __restrict__ tok, int window) {
  const int64_t t = blockIdx.x;
  const int b = tok[2 * t], pos = tok[2 * t + 1];
  const int slot = seq[4 * b], pos0 = seq[4 * b + 1], n = seq[4 * b + 2];
  if (pos < pos0 + n - window) return;          // a later row of this step takes the same ring row
  const T* src = qkv + t * stride + nq;
  const int64_t row = static_cast<int64_t>(slot) * window + pos % window;
  for (int c = threadIdx.x; c < nk; c += NT) kc[row * nk + c] = src[c];
  for (int c = threadIdx.x; c < nv; c += NT) vc[row * nv + c] = src[nk + c];
}

bool act_ok(int act) { return act == GBXM_BF16 || act == GBXM_F32; }

}  // namespace
}  // namespace gbxm

using namespace gbxm;

extern "C" {

int gbxm_version(void) { return 100; }
const char* gbxm_last_error(void) { return g_err; }

#define GBXM_DISPATCH(act, CALL)              \
  do {                                        \
    if ((act) == GBXM_BF16) { using T = bf16_t; CALL; } else { using T = float; CALL; } \
  } while (0)

int gbxm_embed_scaled(const void* table, const int64_t* tokens, float* x, void* h, int64_t T_, int32_t width, float scale, int32_t act,
                      void* stream) {
  if (!act_ok(act) || !table || !tokens || !x || width <= 0 || T_ < 0) return fail(GBXM_ERR_INVALID, "embed_scaled: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (embed_kernel<T><<<dim3(T_), NT, 0, s>>>(static_cast<const T*>(table), tokens, x, static_cast<T*>(h), width, scale)));
  return after_launch("embed_scaled");
}

int gbxm_segment_rmsnorm(void* rows, int64_t T_, int64_t row_stride, int32_t n0, int32_t n1, const float* w0, const float* w1, float eps,
                         int32_t act, void* stream) {
  if (!act_ok(act) || !rows || !w0 || !w1 || n0 <= 0 || n1 <= 0 || row_stride < n0 + n1 || T_ < 0)
    return fail(GBXM_ERR_INVALID, "segment_rmsnorm: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (segment_rmsnorm_kernel<T><<<dim3(T_, 2), NT, 0, s>>>(static_cast<T*>(rows), row_stride, n0, n1, w0, w1, eps)));
  return after_launch("segment_rmsnorm");
}

int gbxm_residual_norm_add(float* x, const void* branch, const float* mix, const float* w, void* h, int64_t T_, int32_t width, int32_t top,
                           float eps, float mult, int32_t act, void* stream) {
  if (!act_ok(act) || !x || !branch || !w || width <= 0 || top < 1 || T_ < 0 || (top > 1 && !mix))
    return fail(GBXM_ERR_INVALID, "residual_norm_add: bad argument");
  if (act == GBXM_BF16 && !h) return fail(GBXM_ERR_INVALID, "residual_norm_add: bf16 needs the image buffer");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (residual_norm_add_kernel<T><<<dim3(T_), NT, 0, s>>>(x, static_cast<const T*>(branch), mix, w, static_cast<T*>(h), width,
                                                                            top, eps, mult)));
  return after_launch("residual_norm_add");
}

int gbxm_stream_rmsnorm(const float* x, const float* w, void* out, int64_t T_, int32_t width, float eps, int32_t act, void* stream) {
  if (!act_ok(act) || !x || !w || !out || width <= 0 || T_ < 0) return fail(GBXM_ERR_INVALID, "stream_rmsnorm: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (stream_rmsnorm_kernel<T><<<dim3(T_), NT, 0, s>>>(x, w, static_cast<T*>(out), width, eps)));
  return after_launch("stream_rmsnorm");
}

int gbxm_route_topk(const float* logits, int32_t* idx, float* weight, int64_t T_, int32_t E, int32_t top, int32_t renorm, void* stream) {
  if (!logits || !idx || !weight || E <= 0 || top < 1 || top > E || T_ < 0) return fail(GBXM_ERR_INVALID, "route_topk: bad argument");
  if (E > 8192) return fail(GBXM_ERR_UNSUPPORTED, "route_topk: more than 8192 experts");
  if (top > NT) return fail(GBXM_ERR_UNSUPPORTED, "route_topk: top > %d", NT);
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  route_topk_kernel<<<dim3(T_), NT, E * sizeof(float), s>>>(logits, idx, weight, E, top, renorm);
  return after_launch("route_topk");
}

int gbxm_window_append(const void* qkv, int64_t row_stride, int32_t nq, int32_t nk, int32_t nv, void* kcache, void* vcache, const int32_t* seq,
                       const int32_t* tok, int64_t T_, int32_t window, int32_t act, void* stream) {
  if (!act_ok(act) || !qkv || !kcache || !vcache || !seq || !tok || nq < 0 || nk <= 0 || nv <= 0 || row_stride < nq + nk + nv || window < 1 ||
      T_ < 0)
    return fail(GBXM_ERR_INVALID, "window_append: bad argument");
  if (T_ == 0) return GBXM_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GBXM_DISPATCH(act, (window_append_kernel<T><<<dim3(T_), NT, 0, s>>>(static_cast<const T*>(qkv), row_stride, nq, nk, nv, static_cast<T*>(kcache),
                                                                        static_cast<T*>(vcache), seq, tok, window)));
  return after_launch("window_append");
}

}  // extern "C"
