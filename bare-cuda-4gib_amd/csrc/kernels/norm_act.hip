// A norm that is added to the residual stream (the second norm of a layer whose sublayers are normed on both
// sides), the xIELU activation, and a gated unit with clamped branches.  One instantiation per storage type; all arithmetic in float.
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kBlock = 256;

__device__ inline float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// x[r, :] += y[r, :] * rsqrt(mean(y[r]^2) + eps) * w.  The row of y is read twice (the second time from the cache).
template <typename TY>
__global__ __launch_bounds__(kBlock) void rmsnorm_add_kernel(float* __restrict__ x, const TY* __restrict__ y,
                                                             const float* __restrict__ w, int hidden, float eps) {
  __shared__ float scratch[16];
  const TY* yr = y + static_cast<size_t>(blockIdx.x) * hidden;
  float* xr = x + static_cast<size_t>(blockIdx.x) * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += kBlock) {
    const float v = to_float(yr[i]);
    ss += v * v;
  }
  const float scale = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(hidden) + eps);
  for (int i = threadIdx.x; i < hidden; i += kBlock) xr[i] += to_float(yr[i]) * scale * w[i];
}

// act(z) = softplus(p) z^2 + z / 2 for z > 0, (1/2 + softplus(q)) (e^z - 1 - z) + z / 2 otherwise.
template <typename T>
__global__ void xielu_kernel(const T* __restrict__ in, T* __restrict__ out, const float* __restrict__ pq, long total) {
  const float ap = softplus_f(pq[0]), aq = 0.5f + softplus_f(pq[1]);
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < total; i += stride) {
    const float z = to_float(in[i]);
    const float r = z > 0.f ? ap * z * z + 0.5f * z : aq * (expm1f(z) - z) + 0.5f * z;
    out[i] = from_float<T>(r);
  }
}

// The same, eight elements a thread in pieces of 16 bytes (bfloat16), for sizes that are whole pieces.
__global__ void xielu_pieces_kernel(const uint4* __restrict__ in, uint4* __restrict__ out, const float* __restrict__ pq, long pieces) {
  const float ap = softplus_f(pq[0]), aq = 0.5f + softplus_f(pq[1]);
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < pieces; i += stride) {
    const uint4 v = in[i];
    unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float z[2] = {__uint_as_float(w[e] << 16), __uint_as_float(w[e] & 0xffff0000u)};
#pragma unroll
      for (int j = 0; j < 2; ++j) z[j] = z[j] > 0.f ? ap * z[j] * z[j] + 0.5f * z[j] : aq * (expm1f(z[j]) - z[j]) + 0.5f * z[j];
      w[e] = static_cast<unsigned>(bf16_bits_from_float(z[0])) | (static_cast<unsigned>(bf16_bits_from_float(z[1])) << 16);
    }
    out[i] = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// out[t, i] = g sigmoid(slope g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit); gu [T, 2 I]: a row's
// gates, then its ups.
template <typename T>
__global__ void clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ out, float limit, float slope, long total, int inter) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < total; i += stride) {
    const long r = i / inter;
    const int c = static_cast<int>(i - r * inter);
    const float g = fminf(to_float(gu[r * 2 * inter + c]), limit);
    const float u = fminf(fmaxf(to_float(gu[r * 2 * inter + inter + c]), -limit), limit);
    out[i] = from_float<T>(g / (1.0f + expf(-slope * g)) * (u + 1.0f));
  }
}

// The same for bfloat16 and I a multiple of 8: a thread takes eight neighbouring outputs, in pieces of 16 bytes.
__global__ void clamped_glu_pieces_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, float limit, float slope,
                                          long pieces, int inter) {
  const int per_row = inter / 8;
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < pieces; i += stride) {
    const long r = i / per_row;
    const int c = static_cast<int>(i - r * per_row) * 8;
    const uint4 gv = *reinterpret_cast<const uint4*>(gu + r * 2 * inter + c);
    const uint4 uv = *reinterpret_cast<const uint4*>(gu + r * 2 * inter + inter + c);
    const unsigned gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    unsigned o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float res[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float g = fminf(__uint_as_float(j ? gw[e] & 0xffff0000u : gw[e] << 16), limit);
        const float u = fminf(fmaxf(__uint_as_float(j ? uw[e] & 0xffff0000u : uw[e] << 16), -limit), limit);
        res[j] = g / (1.0f + expf(-slope * g)) * (u + 1.0f);
      }
      o[e] = static_cast<unsigned>(bf16_bits_from_float(res[0])) | (static_cast<unsigned>(bf16_bits_from_float(res[1])) << 16);
    }
    *reinterpret_cast<uint4*>(out + r * inter + c) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

// z Phi(z), the exact gelu: 0.5 z (1 + erf(z / sqrt 2)).
template <typename T>
__global__ void gelu_kernel(const T* __restrict__ in, T* __restrict__ out, long total) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < total; i += stride) {
    const float z = to_float(in[i]);
    out[i] = from_float<T>(0.5f * z * (1.0f + erff(z * 0.70710678118654752440f)));
  }
}

int grid_for(long total) {
  const long g = (total + kBlock - 1) / kBlock;
  return static_cast<int>(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

// out[t] = h[t] + (h[t - 1] - h[t]) * mix with h = (x * rsqrt(mean(x^2) + eps) * w rounded to the output's type): an RMS
// norm and the token shift behind it in one pass.  A workgroup is one row; it works out the row before once more from
// the stream (that row is in the cache) instead of waiting for it.  A request's first row of the step reads its state
// (the h of its last row so far; zeros when it was admitted), and the same workgroup -- so nobody reads what another
// writes -- leaves the h of the request's last row of this step there.  V elements a thread and trip (4 where the width
// and the addresses allow: 16-byte loads, all of a pass in flight together).
template <int V> struct Pack { float v[V]; };
template <int V> __device__ inline Pack<V> load_pack(const float* p) {
  Pack<V> r;
  if (V == 4) { const float4 f = *reinterpret_cast<const float4*>(p); r.v[0] = f.x, r.v[1 % V] = f.y, r.v[2 % V] = f.z, r.v[3 % V] = f.w; }
  else r.v[0] = p[0];
  return r;
}
template <int V> __device__ inline Pack<V> load_pack(const bf16_t* p) {
  Pack<V> r;
  if (V == 4) {
    const uint2 b = *reinterpret_cast<const uint2*>(p);
    r.v[0] = __uint_as_float(b.x << 16), r.v[1 % V] = __uint_as_float(b.x & 0xffff0000u);
    r.v[2 % V] = __uint_as_float(b.y << 16), r.v[3 % V] = __uint_as_float(b.y & 0xffff0000u);
  } else r.v[0] = to_float(p[0]);
  return r;
}
template <int V> __device__ inline void store_pack(float* p, const Pack<V>& r) {
  if (V == 4) *reinterpret_cast<float4*>(p) = make_float4(r.v[0], r.v[1 % V], r.v[2 % V], r.v[3 % V]);
  else p[0] = r.v[0];
}
template <int V> __device__ inline void store_pack(bf16_t* p, const Pack<V>& r) {
  if (V == 4) {
    uint2 b;
    b.x = bf16_bits_from_float(r.v[0]) | (static_cast<uint32_t>(bf16_bits_from_float(r.v[1 % V])) << 16);
    b.y = bf16_bits_from_float(r.v[2 % V]) | (static_cast<uint32_t>(bf16_bits_from_float(r.v[3 % V])) << 16);
    *reinterpret_cast<uint2*>(p) = b;
  } else p[0] = from_float<bf16_t>(r.v[0]);
}

template <typename TO, int V>
__global__ __launch_bounds__(kBlock) void rmsnorm_shift_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                               const float* __restrict__ mix, TO* __restrict__ out,
                                                               TO* __restrict__ state, const int32_t* __restrict__ row_seq,
                                                               const int32_t* __restrict__ seq_start,
                                                               const int32_t* __restrict__ seq_slots, int hidden, float eps) {
  __shared__ float scratch[3][16];
  const int row = blockIdx.x, seq = row_seq[row];
  const int first = seq_start[seq], last = seq_start[seq + 1] - 1;
  const bool from_state = row == first;                     // (the same for every thread of the workgroup)
  const float* xr = x + static_cast<size_t>(row) * hidden;
  const float* xo = from_state ? x + static_cast<size_t>(last) * hidden : xr - hidden;   // the other row this workgroup norms
  const bool other = !from_state || last != row;
  float ss = 0.f, so = 0.f;
#pragma unroll 4
  for (int i = V * threadIdx.x; i < hidden; i += V * kBlock) {
    const Pack<V> a = load_pack<V>(xr + i), b = other ? load_pack<V>(xo + i) : a;
#pragma unroll
    for (int e = 0; e < V; ++e) ss = fmaf(a.v[e], a.v[e], ss), so = fmaf(b.v[e], b.v[e], so);
  }
  const float rs = 1.0f / sqrtf(block_sum(ss, scratch[0]) / static_cast<float>(hidden) + eps);
  const float ro = 1.0f / sqrtf(block_sum(so, scratch[1]) / static_cast<float>(hidden) + eps);
  TO* st = state + static_cast<size_t>(seq_slots[seq]) * hidden;
  TO* orow = out + static_cast<size_t>(row) * hidden;
#pragma unroll 4
  for (int i = V * threadIdx.x; i < hidden; i += V * kBlock) {
    const Pack<V> a = load_pack<V>(xr + i), b = other ? load_pack<V>(xo + i) : a, wi = load_pack<V>(w + i), mi = load_pack<V>(mix + i);
    Pack<V> before, h, o, keep;
    if (from_state) before = load_pack<V>(st + i);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      h.v[e] = to_float(from_float<TO>(a.v[e] * rs * wi.v[e]));
      const float ho = to_float(from_float<TO>(b.v[e] * ro * wi.v[e]));      // the row before, or the request's last
      if (!from_state) before.v[e] = ho;
      o.v[e] = fmaf(before.v[e] - h.v[e], mi.v[e], h.v[e]);
      keep.v[e] = ho;
    }
    if (from_state) store_pack<V>(st + i, keep);
    store_pack<V>(orow + i, o);
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_rmsnorm_add(float* x, const void* y, int y_dtype, const float* w, int n_rows, int hidden, float eps,
                                void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && hidden > 0 && x && y && w, "rmsnorm_add: bad arguments rows=%d H=%d", n_rows, hidden);
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (y_dtype == kF32) rmsnorm_add_kernel<float><<<n_rows, kBlock, 0, s>>>(x, static_cast<const float*>(y), w, hidden, eps);
  else if (y_dtype == kBF16) rmsnorm_add_kernel<bf16_t><<<n_rows, kBlock, 0, s>>>(x, static_cast<const bf16_t*>(y), w, hidden, eps);
  else return fail("rmsnorm_add: unknown dtype %d", y_dtype);
  return check_launch("rmsnorm_add");
}

extern "C" int bc4g_xielu(const void* in, void* out, int dtype, const float* pq, long total, void* stream) {
  BC4G_REQUIRE(total >= 0 && in && out && pq, "xielu: bad arguments (%ld elements)", total);
  if (total == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32) xielu_kernel<float><<<grid_for(total), kBlock, 0, s>>>(static_cast<const float*>(in), static_cast<float*>(out), pq, total);
  else if (dtype == kBF16 && total % 8 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0)
    xielu_pieces_kernel<<<grid_for(total / 8), kBlock, 0, s>>>(static_cast<const uint4*>(in), static_cast<uint4*>(out), pq, total / 8);
  else if (dtype == kBF16) xielu_kernel<bf16_t><<<grid_for(total), kBlock, 0, s>>>(static_cast<const bf16_t*>(in), static_cast<bf16_t*>(out), pq, total);
  else return fail("xielu: unknown dtype %d", dtype);
  return check_launch("xielu");
}

extern "C" int bc4g_clamped_glu(const void* gu, void* out, int dtype, float limit, float slope, int n_rows, int inter, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && inter > 0 && gu && out && gu != out, "clamped_glu: bad arguments rows=%d I=%d", n_rows, inter);
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long total = static_cast<long>(n_rows) * inter;
  if (dtype == kF32) clamped_glu_kernel<float><<<grid_for(total), kBlock, 0, s>>>(static_cast<const float*>(gu), static_cast<float*>(out), limit, slope, total, inter);
  else if (dtype == kBF16 && inter % 8 == 0 && reinterpret_cast<uintptr_t>(gu) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0)
    clamped_glu_pieces_kernel<<<grid_for(total / 8), kBlock, 0, s>>>(static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), limit, slope, total / 8, inter);
  else if (dtype == kBF16) clamped_glu_kernel<bf16_t><<<grid_for(total), kBlock, 0, s>>>(static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), limit, slope, total, inter);
  else return fail("clamped_glu: unknown dtype %d", dtype);
  return check_launch("clamped_glu");
}

extern "C" int bc4g_gelu(const void* in, void* out, int dtype, long total, void* stream) {
  BC4G_REQUIRE(total >= 0 && in && out, "gelu: bad arguments total=%ld", total);
  if (total == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32) gelu_kernel<float><<<grid_for(total), kBlock, 0, s>>>(static_cast<const float*>(in), static_cast<float*>(out), total);
  else if (dtype == kBF16) gelu_kernel<bf16_t><<<grid_for(total), kBlock, 0, s>>>(static_cast<const bf16_t*>(in), static_cast<bf16_t*>(out), total);
  else return fail("gelu: unknown dtype %d", dtype);
  return check_launch("gelu");
}

extern "C" int bc4g_rmsnorm_shift(const float* x, const float* w, const float* mix, void* out, void* state, int dtype,
                                  const int32_t* row_seq, const int32_t* seq_start, const int32_t* seq_slots, int n_rows,
                                  int hidden, float eps, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && hidden > 0 && x && w && mix && out && state && row_seq && seq_start && seq_slots,
               "rmsnorm_shift: bad arguments rows=%d H=%d", n_rows, hidden);
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool four = hidden % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(mix) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                    reinterpret_cast<uintptr_t>(state) % 16 == 0;
#define BC4G_SHIFT(T, V)                                                                                                    \
  rmsnorm_shift_kernel<T, V><<<n_rows, kBlock, 0, s>>>(x, w, mix, static_cast<T*>(out), static_cast<T*>(state), row_seq, seq_start, \
                                                      seq_slots, hidden, eps)
  if (dtype == kF32) { if (four) BC4G_SHIFT(float, 4); else BC4G_SHIFT(float, 1); }
  else if (dtype == kBF16) { if (four) BC4G_SHIFT(bf16_t, 4); else BC4G_SHIFT(bf16_t, 1); }
  else return fail("rmsnorm_shift: unknown dtype %d", dtype);
#undef BC4G_SHIFT
  return check_launch("rmsnorm_shift");
}
