// A mixture of experts' router and the activation of its experts side by side.
//
//   route       per row: s = softmax(logits) over all experts (float32); the choice goes by s + correction; the experts lie in
//               equal groups of neighbours, a group counts by its largest choice, and only the best groups' experts can be
//               chosen (the others count as minus infinity, not as zero: a choice may be negative); the largest `top`
//               choices win, the lower index among equals.  Out: a row of weights over all experts -- s of the chosen, as
//               it is, zero elsewhere -- and the chosen experts' indices.
//               With `squash` s = sigmoid(logit), every expert by itself; with `normalize` the chosen experts' weights are
//               their s divided by the sum of the chosen s (+ 1e-20); the weights are multiplied by a factor last.
//   routed_gelu every expert's plain unit (the exact gelu) on its part of one wide product's row, times the row's weight for
//               that expert; a shared unit at the end counts as it is.
//   routed_glu  every expert's clamped gated unit on its part of one wide product's row, times the row's weight for that
//               expert (zero for the experts the row did not choose), and a shared unit with a gate per row at the end:
//               what one product over all experts' down matrices then adds up is the weighted sum of the chosen experts.
#include <float.h>
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kMaxExperts = 1024;
constexpr int kBlock = 256;

// One wave a row.
__global__ __launch_bounds__(kWave) void moe_route_kernel(const float* __restrict__ logits, long logits_row,
                                                          const float* __restrict__ correction, float* __restrict__ weights,
                                                          int32_t* __restrict__ chosen, int experts, int groups, int keep, int top,
                                                          int squash, int normalize, float factor) {
  __shared__ float s_s[kMaxExperts];        // the scores
  __shared__ float c_s[kMaxExperts];        // the choices (minus infinity once taken, or outside the kept groups)
  __shared__ float g_s[kMaxExperts];        // the groups' largest choices
  const int row = blockIdx.x, lane = threadIdx.x;
  const float* z = logits + row * logits_row;
  float sum = 1.0f;
  if (squash) {
    for (int e = lane; e < experts; e += kWave) s_s[e] = 1.0f / (1.0f + expf(-z[e]));
  } else {
    float top_z = -INFINITY;
    for (int e = lane; e < experts; e += kWave) top_z = fmaxf(top_z, z[e]);
    top_z = wave_max(top_z);
    sum = 0.f;
    for (int e = lane; e < experts; e += kWave) {
      const float p = expf(z[e] - top_z);
      s_s[e] = p;
      sum += p;
    }
    sum = wave_sum(sum);
  }
  const int per = experts / groups;
  for (int e = lane; e < experts; e += kWave) {
    const float s = s_s[e] / sum;
    s_s[e] = s;
    c_s[e] = correction ? s + correction[e] : s;
    weights[static_cast<long>(row) * experts + e] = 0.f;
  }
  __syncthreads();
  for (int g = lane; g < groups; g += kWave) {
    float best = -INFINITY;
    for (int i = 0; i < per; ++i) best = fmaxf(best, c_s[g * per + i]);
    g_s[g] = best;
  }
  __syncthreads();
  // an expert stays if fewer than `keep` groups come before its group (larger, or equal with a lower index)
  for (int g = lane; g < groups; g += kWave) {
    const float mine = g_s[g];
    int before = 0;
    for (int o = 0; o < groups; ++o) before += (g_s[o] > mine || (g_s[o] == mine && o < g)) ? 1 : 0;
    if (before >= keep)
      for (int i = 0; i < per; ++i) c_s[g * per + i] = -INFINITY;
  }
  __syncthreads();
  float picked = 0.f;                                          // the chosen experts' scores, added up in the order of choice
  for (int n = 0; n < top; ++n) {
    float best = -INFINITY;
    int at = experts;
    for (int e = lane; e < experts; e += kWave)
      if (c_s[e] > best) best = c_s[e], at = e;               // (ascending e: the lower index among this lane's equals)
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float other = __shfl_xor(best, off, kWave);
      const int other_at = __shfl_xor(at, off, kWave);
      if (other > best || (other == best && other_at < at)) best = other, at = other_at;
    }
    if (at >= experts) break;                                 // fewer experts left than asked for
    picked += s_s[at];
    if (lane == 0) {
      weights[static_cast<long>(row) * experts + at] = s_s[at] * (normalize ? 1.0f : factor);
      if (chosen) chosen[static_cast<long>(row) * top + n] = at;
      c_s[at] = -INFINITY;
    }
    __syncthreads();
  }
  if (normalize) {                                            // (the row's weights are this wave's own writes)
    const float by = factor / (picked + 1e-20f);
    for (int e = lane; e < experts; e += kWave) {
      const float w = weights[static_cast<long>(row) * experts + e];
      if (w != 0.f) weights[static_cast<long>(row) * experts + e] = w * by;
    }
  }
}

__device__ inline float gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }

// PIECE elements a thread (16 bytes), all of one expert: ff and shared_ff are multiples of PIECE (1: any sizes).
template <typename T, int PIECE>
__global__ void routed_gelu_kernel(const T* z, T* out, const float* __restrict__ weights, long total,      // (out may be z)
                                   int experts, int ff, int shared_ff) {
  const int row_width = experts * ff + shared_ff;
  const long stride = static_cast<long>(blockDim.x) * gridDim.x * PIECE;
  for (long i = (blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x) * PIECE; i < total; i += stride) {
    const long r = i / row_width;
    const int c = static_cast<int>(i - r * row_width);
    const float w = c < experts * ff ? weights[r * experts + c / ff] : 1.0f;
    if (PIECE == 1) {
      out[i] = from_float<T>(w != 0.f ? w * gelu_erf(to_float(z[i])) : 0.f);
    } else {
      __align__(16) T piece[PIECE];
      *reinterpret_cast<uint4*>(piece) = w != 0.f ? *reinterpret_cast<const uint4*>(z + i) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int e = 0; e < PIECE; ++e) piece[e] = from_float<T>(w != 0.f ? w * gelu_erf(to_float(piece[e])) : 0.f);
      *reinterpret_cast<uint4*>(out + i) = *reinterpret_cast<const uint4*>(piece);
    }
  }
}

template <typename T>
__global__ void routed_glu_kernel(const T* __restrict__ gu, T* __restrict__ out, const float* __restrict__ weights,
                                  const float* __restrict__ shared_logit, long shared_row, float limit, float shared_limit,
                                  float slope, long total, int experts, int ff, int shared_ff) {
  const int out_row = experts * ff + shared_ff;
  const long in_row = 2L * out_row;
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < total; i += stride) {
    const long r = i / out_row;
    const int c = static_cast<int>(i - r * out_row);
    float w, lim;
    long g_at;
    int width;
    if (c < experts * ff) {
      const int e = c / ff;
      w = weights[r * experts + e];
      g_at = r * in_row + 2L * e * ff + (c - e * ff);
      width = ff, lim = limit;
    } else {
      w = 1.0f / (1.0f + expf(-shared_logit[r * shared_row]));
      g_at = r * in_row + 2L * experts * ff + (c - experts * ff);
      width = shared_ff, lim = shared_limit;
    }
    float y = 0.f;
    if (w != 0.f) {
      const float g = fminf(to_float(gu[g_at]), lim);
      const float u = fminf(fmaxf(to_float(gu[g_at + width]), -lim), lim);
      y = w * (g / (1.0f + expf(-slope * g)) * (u + 1.0f));
    }
    out[i] = from_float<T>(y);
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_moe_route(const float* logits, long logits_row, const float* correction, float* weights, int32_t* chosen,
                              int n_rows, int experts, int groups, int keep, int top, int squash, int normalize, float factor,
                              void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && experts > 0 && experts <= kMaxExperts && logits && weights && logits_row >= experts,
               "moe_route: bad arguments rows=%d experts=%d (at most %d)", n_rows, experts, kMaxExperts);
  BC4G_REQUIRE(groups > 0 && experts % groups == 0 && keep > 0 && keep <= groups && top > 0 && top <= experts,
               "moe_route: %d experts in %d groups of which %d are kept, %d chosen", experts, groups, keep, top);
  if (n_rows == 0) return 0;
  moe_route_kernel<<<n_rows, kWave, 0, static_cast<hipStream_t>(stream)>>>(logits, logits_row, correction, weights, chosen,
                                                                           experts, groups, keep, top, squash, normalize,
                                                                           factor);
  return check_launch("moe_route");
}

extern "C" int bc4g_routed_gelu(const void* z, void* out, int dtype, const float* weights, int n_rows, int experts, int ff,
                                int shared_ff, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && experts >= 0 && ff >= 0 && shared_ff >= 0 && experts * ff + shared_ff > 0 && z && out,
               "routed_gelu: bad arguments rows=%d experts=%d ff=%d shared=%d", n_rows, experts, ff, shared_ff);
  BC4G_REQUIRE(experts == 0 || weights, "routed_gelu: the weights are missing");
  const long total = static_cast<long>(n_rows) * (static_cast<long>(experts) * ff + shared_ff);
  if (total == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int piece = dtype == kF32 ? 4 : 8;      // elements in 16 bytes
  const bool pieces = ff % piece == 0 && shared_ff % piece == 0 && reinterpret_cast<uintptr_t>(z) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const long threads = pieces ? total / piece : total;
  const long blocks = (threads + kBlock - 1) / kBlock;
  const int grid = static_cast<int>(blocks > 65535 ? 65535 : blocks);
#define BC4G_ROUTED_GELU(T, P)                                                                                              \
  routed_gelu_kernel<T, P><<<grid, kBlock, 0, s>>>(static_cast<const T*>(z), static_cast<T*>(out), weights, total, experts, ff, shared_ff)
  if (dtype == kF32) {
    if (pieces) BC4G_ROUTED_GELU(float, 4); else BC4G_ROUTED_GELU(float, 1);
  } else if (dtype == kBF16) {
    if (pieces) BC4G_ROUTED_GELU(bf16_t, 8); else BC4G_ROUTED_GELU(bf16_t, 1);
  } else {
    return fail("routed_gelu: unknown dtype %d", dtype);
  }
#undef BC4G_ROUTED_GELU
  return check_launch("routed_gelu");
}

extern "C" int bc4g_routed_glu(const void* gu, void* out, int dtype, const float* weights, const float* shared_logit,
                               long shared_row, float limit, float shared_limit, float slope, int n_rows, int experts, int ff,
                               int shared_ff, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && experts >= 0 && ff >= 0 && shared_ff >= 0 && experts * ff + shared_ff > 0 && gu && out && gu != out,
               "routed_glu: bad arguments rows=%d experts=%d ff=%d shared=%d", n_rows, experts, ff, shared_ff);
  BC4G_REQUIRE((experts == 0 || weights) && (shared_ff == 0 || shared_logit), "routed_glu: the weights or the shared gate are missing");
  const long total = static_cast<long>(n_rows) * (static_cast<long>(experts) * ff + shared_ff);
  if (total == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long blocks = (total + kBlock - 1) / kBlock;
  const int grid = static_cast<int>(blocks > 65535 ? 65535 : blocks);
  if (dtype == kF32)
    routed_glu_kernel<float><<<grid, kBlock, 0, s>>>(static_cast<const float*>(gu), static_cast<float*>(out), weights, shared_logit,
                                                     shared_row, limit, shared_limit, slope, total, experts, ff, shared_ff);
  else if (dtype == kBF16)
    routed_glu_kernel<bf16_t><<<grid, kBlock, 0, s>>>(static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), weights,
                                                      shared_logit, shared_row, limit, shared_limit, slope, total, experts, ff,
                                                      shared_ff);
  else
    return fail("routed_glu: unknown dtype %d", dtype);
  return check_launch("routed_glu");
}
