// What happens to the float32 residual stream between two sublayers, in one launch:
//
//   update   x = (keep ? x : 0) + s * y + b      y a sublayer's float32 output, s and b one number a channel (each may be
//            absent: 1 and 0), all element by element in float32; x is written back
//   norm     and, if a weight is given, out = N(x) in the activations' dtype for whoever reads the stream next:
//            the row in `groups` equal runs of neighbouring channels, a run r scaled by 1 / sqrt(mean(r^2) + eps) of its own,
//            then every channel times its weight
//   beside   out[t] = [x[t] | table[ids[t]] * factor] in the activations' dtype: the stream and the embedding of the
//            same token side by side, the operand of a product over both
//
// A workgroup is one part of one row; a thread keeps its elements in registers between the sum and the scaling where the
// part has at most 256 * 4 * kHeld elements, and reads x back otherwise.  The order of a part's sum depends on the
// part's width alone.
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kBlock = 256;
constexpr int kHeld = 4;      // pieces of four a thread keeps

template <typename TW, typename TO, bool HELD>
__global__ __launch_bounds__(kBlock) void stream_update_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                               const float* __restrict__ s, const float* __restrict__ b, int keep,
                                                               const TW* __restrict__ w, TO* __restrict__ out, int part, int groups,
                                                               float eps) {
  __shared__ float scratch[16];
  const size_t at = static_cast<size_t>(blockIdx.x) * part;
  const int col0 = static_cast<int>(blockIdx.x % groups) * part;
  float* xr = x + at;
  const float* yr = y + at;
  float held[kHeld][4];
  float ss = 0.f;
  if (HELD) {      // part a multiple of 4: pieces of four
#pragma unroll
    for (int c = 0; c < kHeld; ++c) {
      const int i = (c * kBlock + threadIdx.x) * 4;
      if (i < part) {
        const float4 yv = *reinterpret_cast<const float4*>(yr + i);
        float v[4] = {yv.x, yv.y, yv.z, yv.w};
        if (s) {
          const float4 sv = *reinterpret_cast<const float4*>(s + col0 + i);
          v[0] *= sv.x, v[1] *= sv.y, v[2] *= sv.z, v[3] *= sv.w;
        }
        if (keep) {
          const float4 xv = *reinterpret_cast<const float4*>(xr + i);
          v[0] += xv.x, v[1] += xv.y, v[2] += xv.z, v[3] += xv.w;
        }
        if (b) {
          const float4 bv = *reinterpret_cast<const float4*>(b + col0 + i);
          v[0] += bv.x, v[1] += bv.y, v[2] += bv.z, v[3] += bv.w;
        }
        *reinterpret_cast<float4*>(xr + i) = make_float4(v[0], v[1], v[2], v[3]);
#pragma unroll
        for (int e = 0; e < 4; ++e) held[c][e] = v[e], ss = fmaf(v[e], v[e], ss);
      }
    }
  } else {
    for (int i = threadIdx.x; i < part; i += kBlock) {
      float v = yr[i];
      if (s) v *= s[col0 + i];
      if (keep) v += xr[i];
      if (b) v += b[col0 + i];
      xr[i] = v;
      ss = fmaf(v, v, ss);
    }
  }
  if (!w) return;
  const float scale = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(part) + eps);
  TO* orow = out + at;
  if (HELD) {
#pragma unroll
    for (int c = 0; c < kHeld; ++c) {
      const int i = (c * kBlock + threadIdx.x) * 4;
      if (i < part) {
#pragma unroll
        for (int e = 0; e < 4; ++e) orow[i + e] = from_float<TO>(held[c][e] * scale * to_float(w[col0 + i + e]));
      }
    }
  } else {
    for (int i = threadIdx.x; i < part; i += kBlock)      // (a thread reads back what it wrote itself)
      orow[i] = from_float<TO>(xr[i] * scale * to_float(w[col0 + i]));
  }
}

template <typename TT, typename TO>
__global__ void embed_beside_kernel(const float* __restrict__ x, const TT* __restrict__ table, const int32_t* __restrict__ ids,
                                    float factor, TO* __restrict__ out, int hidden) {
  const size_t row = blockIdx.x;
  const float* xr = x + row * hidden;
  const TT* src = table + static_cast<size_t>(ids[row]) * hidden;
  TO* dst = out + row * 2 * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    dst[i] = from_float<TO>(xr[i]);
    dst[hidden + i] = from_float<TO>(to_float(src[i]) * factor);
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_stream_update(float* x, const float* y, const float* scale, const float* bias, int keep, const void* w,
                                  int w_dtype, void* out, int out_dtype, int n_rows, int width, int groups, float eps,
                                  void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && width > 0 && groups > 0 && width % groups == 0 && static_cast<long>(n_rows) * groups < (1L << 31),
               "stream_update: bad sizes rows=%d H=%d in %d groups", n_rows, width, groups);
  BC4G_REQUIRE(x && y && x != y && ((w == nullptr) == (out == nullptr)), "stream_update: a tensor is missing, or the norm has a weight and no room");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int part = width / groups, blocks = n_rows * groups;
  const bool held = part % 4 == 0 && part <= kBlock * 4 * kHeld;
#define BC4G_UPDATE(TW, TO)                                                                                                   \
  do {                                                                                                                        \
    if (held) stream_update_kernel<TW, TO, true><<<blocks, kBlock, 0, s>>>(x, y, scale, bias, keep, static_cast<const TW*>(w), \
                                                                           static_cast<TO*>(out), part, groups, eps);           \
    else stream_update_kernel<TW, TO, false><<<blocks, kBlock, 0, s>>>(x, y, scale, bias, keep, static_cast<const TW*>(w),     \
                                                                       static_cast<TO*>(out), part, groups, eps);               \
  } while (0)
  if (!w) BC4G_UPDATE(float, float);
  else if (w_dtype == kF32 && out_dtype == kF32) BC4G_UPDATE(float, float);
  else if (w_dtype == kF32 && out_dtype == kBF16) BC4G_UPDATE(float, bf16_t);
  else if (w_dtype == kBF16 && out_dtype == kF32) BC4G_UPDATE(bf16_t, float);
  else if (w_dtype == kBF16 && out_dtype == kBF16) BC4G_UPDATE(bf16_t, bf16_t);
  else return fail("stream_update: unknown dtypes w=%d out=%d", w_dtype, out_dtype);
#undef BC4G_UPDATE
  return check_launch("stream_update");
}

extern "C" int bc4g_embed_beside(const float* x, const void* table, int table_dtype, const int32_t* ids, float factor, void* out,
                                 int out_dtype, int n_tokens, int hidden, int vocab, void* stream) {
  BC4G_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0 && x && table && ids && out, "embed_beside: bad arguments T=%d H=%d V=%d",
               n_tokens, hidden, vocab);
  if (n_tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define BC4G_BESIDE(TT, TO)                                                                                                  \
  embed_beside_kernel<TT, TO><<<n_tokens, kBlock, 0, s>>>(x, static_cast<const TT*>(table), ids, factor, static_cast<TO*>(out), hidden)
  if (table_dtype == kF32 && out_dtype == kF32) BC4G_BESIDE(float, float);
  else if (table_dtype == kF32 && out_dtype == kBF16) BC4G_BESIDE(float, bf16_t);
  else if (table_dtype == kBF16 && out_dtype == kF32) BC4G_BESIDE(bf16_t, float);
  else if (table_dtype == kBF16 && out_dtype == kBF16) BC4G_BESIDE(bf16_t, bf16_t);
  else return fail("embed_beside: unknown dtypes table=%d out=%d", table_dtype, out_dtype);
#undef BC4G_BESIDE
  return check_launch("embed_beside");
}
