// Linear attention with a decayed matrix state per head, and what stands around it:
//
//   state     S_t = diag(a_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t        S [dim, vdim] float32 per request and head
//             a_t is one number per head (retention) or a vector per token made from gate logits z,
//             a = sigmoid(z + bias)^(1/tau) (gated linear attention); no softmax, no denominator.
//   rotation  a table of cosines and sines of position * frequency for the rotate-half pairing (element i with element
//             i + half), the frequencies given by the caller (so any scaling of them is the caller's), both multiplied
//             by an amplitude; angles in double.
//   prepare   per (row, head): + bias, RMS norm over the head with a weight, rotation (either pairing), division by the
//             root mean square after the rotation, a factor -- each optional -- into a dense tensor or into the pages
//             of a cache.
//   finish    per (row, head): o / rms(o) (* weight) * factor * act(gate).
//
// The scan walks a request's rows in chunks of 32, each chunk by workgroups of its own (a thread keeps one column of
// the state, dim numbers, in registers): first every chunk from a zero state (what it adds, and the product of its
// decays), then the states between the chunks in a short sequential pass, then every chunk again from its true
// state, writing outputs.  A request that brings at most one chunk (a decode step) takes the last pass alone, from
// and into its state slot.  A row's sums run over the key channels in ascending order in one thread, whatever the batch.
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kChunk = 32;       // rows of a request that one workgroup walks
constexpr int kStage = 16;       // rows whose q, k and decays lie in LDS at a time
constexpr int kMaxHead = 256;    // elements of a head that prepare and finish take

__device__ inline float load_any(const void* p, int dtype, long idx) {
  return dtype == kF32 ? static_cast<const float*>(p)[idx] : to_float(static_cast<const bf16_t*>(p)[idx]);
}
__device__ inline void store_any(void* p, int dtype, long idx, float v) {
  if (dtype == kF32) static_cast<float*>(p)[idx] = v;
  else static_cast<bf16_t*>(p)[idx] = from_float<bf16_t>(v);
}

__global__ void rotary_table_kernel(const int32_t* __restrict__ positions, const double* __restrict__ freqs, double amp,
                                    float* __restrict__ out, long total, int half) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const double angle = static_cast<double>(positions[idx / half]) * freqs[idx % half];
    double sn, cs;
    sincos(angle, &sn, &cs);
    out[2 * idx] = static_cast<float>(cs * amp);
    out[2 * idx + 1] = static_cast<float>(sn * amp);
  }
}

// One wave per (row, head); the heads of up to four sections of one step's rows in one launch (the queries, keys and
// values of an attention layer, say), each section with its own input, size, bias, norm, rotation, factor and output.
struct PrepareSections {
  bc4g_prepare_section s[4];
  int n;
};

__global__ __launch_bounds__(kWave) void heads_prepare_kernel(const PrepareSections all) {
  __shared__ float vals[kMaxHead];
  const int row = blockIdx.x, lane = threadIdx.x;
  int head = blockIdx.y, which = 0;
  while (which + 1 < all.n && head >= all.s[which].heads) head -= all.s[which].heads, ++which;
  const bc4g_prepare_section& p = all.s[which];
  const int dim = p.dim, half = p.half;
  const float* bias = p.bias;
  const float* norm_w = p.norm_w;
  const float* table = p.table;
  float ss = 0.f;
  for (int c = lane; c < dim; c += kWave) {
    float v = load_any(p.in, p.in_dtype, row * p.in_row + static_cast<long>(head) * dim + c);
    if (bias) v += bias[static_cast<long>(head) * dim + c];
    vals[c] = v;
    ss = fmaf(v, v, ss);
  }
  float scale = 1.0f;
  if (norm_w && p.norm_rows) {      // the mean square of the whole row, all heads at once; the weight spans the row too
    const int width = p.heads * dim;
    float all = 0.f;
    const bf16_t* row16 = static_cast<const bf16_t*>(p.in) + row * p.in_row;
    const float* row32 = static_cast<const float*>(p.in) + row * p.in_row;
    // (which way the sum is taken depends on the section alone, never on the row: every row's base is aligned or none is)
    const bool aligned = reinterpret_cast<uintptr_t>(p.in) % 16 == 0 && p.in_row % 8 == 0;
    if (!bias && p.in_dtype == kBF16 && width % 8 == 0 && aligned) {
      // every wave of the row reads the whole row for this sum: in 16-byte pieces, eight elements a lane
      for (int c = lane * 8; c < width; c += kWave * 8) {
        const uint4 bits = *reinterpret_cast<const uint4*>(row16 + c);
        const uint32_t w4[4] = {bits.x, bits.y, bits.z, bits.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float lo = __uint_as_float(w4[e] << 16), hi = __uint_as_float(w4[e] & 0xffff0000u);
          all = fmaf(lo, lo, all), all = fmaf(hi, hi, all);
        }
      }
    } else if (!bias && p.in_dtype == kF32 && width % 4 == 0 && aligned) {
      for (int c = lane * 4; c < width; c += kWave * 4) {
        const float4 v = *reinterpret_cast<const float4*>(row32 + c);
        all = fmaf(v.x, v.x, all), all = fmaf(v.y, v.y, all), all = fmaf(v.z, v.z, all), all = fmaf(v.w, v.w, all);
      }
    } else {
      for (int c = lane; c < width; c += kWave) {
        float v = load_any(p.in, p.in_dtype, row * p.in_row + c);
        if (bias) v += bias[c];
        all = fmaf(v, v, all);
      }
    }
    scale = 1.0f / sqrtf(wave_sum(all) / static_cast<float>(width) + p.eps);
    norm_w += static_cast<long>(head) * dim;
  } else if (norm_w) {
    scale = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(dim) + p.eps);
  }
  __syncthreads();
  long base;
  if (p.slot_map) {
    const long slot = p.slot_map[row];
    base = (slot / p.page_tokens) * p.page_stride + head * p.head_stride + (slot % p.page_tokens) * p.token_stride;
  } else {
    base = row * p.out_row + static_cast<long>(head) * dim;
  }
  float turned[kMaxHead / kWave];      // this lane's elements after norm and rotation
  float ss_after = 0.f;
#pragma unroll
  for (int n = 0; n < kMaxHead / kWave; ++n) {
    const int c = lane + n * kWave;
    float v = 0.f;
    if (c < dim) {
      if (c < 2 * half) {
        // the pair's two members: element i with element i + half, or (neighbours) element 2i with element 2i + 1
        const int i = p.pairing ? c / 2 : (c < half ? c : c - half);
        const int at_lo = p.pairing ? 2 * i : i, at_hi = p.pairing ? 2 * i + 1 : i + half;
        float lo = vals[at_lo] * scale, hi = vals[at_hi] * scale;
        if (norm_w) lo *= norm_w[at_lo], hi *= norm_w[at_hi];
        const float cs = table[(static_cast<long>(row) * half + i) * 2], sn = table[(static_cast<long>(row) * half + i) * 2 + 1];
        v = c == at_lo ? lo * cs - hi * sn : hi * cs + lo * sn;
      } else {
        v = vals[c] * scale;
        if (norm_w) v *= norm_w[c];
      }
    }
    turned[n] = v;
    ss_after = fmaf(v, v, ss_after);
  }
  // (unit_after: the head divided by its root mean square as it stands after the rotation, no weight)
  const float last = p.unit_after ? p.factor / sqrtf(wave_sum(ss_after) / static_cast<float>(dim) + p.eps) : p.factor;
#pragma unroll
  for (int n = 0; n < kMaxHead / kWave; ++n) {
    const int c = lane + n * kWave;
    if (c < dim) store_any(p.out, p.out_dtype, base + c, turned[n] * last);
  }
}

__device__ inline float act_of(float z, int act) {
  if (act == 1) return z / (1.0f + expf(-z));          // silu
  if (act == 2) return 1.0f / (1.0f + expf(-z));        // sigmoid
  return 1.0f;
}

// One wave per (row, head): out = o / rms(o) (* w) * factor * act(gate).
__global__ __launch_bounds__(kWave) void heads_finish_kernel(
    const float* __restrict__ o, const float* __restrict__ w, float eps, float factor, const void* __restrict__ gate,
    int gate_dtype, long gate_row, int act, void* __restrict__ out, int out_dtype, int heads, int vdim) {
  const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + (static_cast<long>(row) * heads + head) * vdim;
  float vals[kMaxHead / kWave];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxHead / kWave; ++i) {
    const int c = lane + i * kWave;
    vals[i] = c < vdim ? orow[c] : 0.f;
    ss = fmaf(vals[i], vals[i], ss);
  }
  const float scale = factor / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps);
#pragma unroll
  for (int i = 0; i < kMaxHead / kWave; ++i) {
    const int c = lane + i * kWave;
    if (c >= vdim) break;
    float v = vals[i] * scale;
    if (w) v *= w[c];
    if (gate) v *= act_of(load_any(gate, gate_dtype, row * gate_row + static_cast<long>(head) * vdim + c), act);
    store_any(out, out_dtype, (static_cast<long>(row) * heads + head) * vdim + c, v);
  }
}

// log(sigmoid(z)) = -softplus(-z)
__device__ inline float log_sigmoid(float z) { return -(fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z)))); }

struct ScanArgs {
  const void* q; int q_dtype; long q_row; float q_scale;
  const void* k; int k_dtype; long k_row;
  const void* v; int v_dtype; long v_row;
  const float* head_decay;                       // [heads], or
  const void* z; int z_dtype; long z_row; const float* z_bias; float inv_tau;      // gate logits [T, heads * dim]
  float* out;                                    // [T, heads, vdim]
  float* state;                                  // [slots, heads, dim, vdim]
  float* chunk_state;                            // [chunks, heads, dim, vdim]: a chunk's sum, then the state before it
  float* chunk_decay;                            // [chunks, heads, dim]
  const int32_t* seq_start; const int32_t* seq_slots; const int32_t* chunk_base;   // [S + 1], [S], [S]
  int heads, dim, vdim;
};

// kPass 0: the chunk from a zero state -> chunk_state, chunk_decay.  kPass 1: the chunk from its true state -> out
// (and, for a request of one chunk, the state slot).  Grid: (vdim / 64, chunks of the longest request, S * heads).
template <int KD, int kPass, bool kPerChannel>
__global__ __launch_bounds__(kWave) void decay_scan_kernel(const ScanArgs a) {
  __shared__ float k_s[kStage][KD];
  __shared__ float q_s[kPass ? kStage : 1][KD];
  __shared__ float a_s[kPerChannel ? kStage : 1][KD];
  const int lane = threadIdx.x, col = blockIdx.x * kWave + lane, chunk = blockIdx.y;
  const int s = blockIdx.z / a.heads, head = blockIdx.z % a.heads;
  const int dim = a.dim, vdim = a.vdim;
  const long start = a.seq_start[s], end = a.seq_start[s + 1];
  const int n_chunks = static_cast<int>((end - start + kChunk - 1) / kChunk);
  const long lo = start + static_cast<long>(chunk) * kChunk, hi = lo + kChunk < end ? lo + kChunk : end;
  if (chunk >= n_chunks || (kPass == 0 && n_chunks < 2)) return;
  const bool live = col < vdim;
  const long per_state = static_cast<long>(dim) * vdim;
  const long slot_at = (static_cast<long>(a.seq_slots[s]) * a.heads + head) * per_state + col;
  const long chunk_id = n_chunks >= 2 ? a.chunk_base[s] + chunk : 0;
  const long chunk_at = (chunk_id * a.heads + head) * per_state + col;
  float S[KD];
  float prod[(KD + kWave - 1) / kWave];       // the chunk's product of decays, channels lane, lane + 64, ...
#pragma unroll
  for (int i = 0; i < (KD + kWave - 1) / kWave; ++i) prod[i] = 1.0f;
  if (kPass == 0) {
#pragma unroll
    for (int d = 0; d < KD; ++d) S[d] = 0.f;
  } else {
    const float* from = n_chunks >= 2 ? a.chunk_state + chunk_at : a.state + slot_at;
#pragma unroll
    for (int d = 0; d < KD; ++d) S[d] = (live && d < dim) ? from[static_cast<long>(d) * vdim] : 0.f;
  }
  const float decay = kPerChannel ? 0.f : a.head_decay[head];
  for (long r0 = lo; r0 < hi; r0 += kStage) {
    const int nr = static_cast<int>(hi - r0 < kStage ? hi - r0 : kStage);
    __syncthreads();
    // Eight elements a lane asked for together (a loop of single loads would wait for each in turn).  The rows lie in
    // LDS KD wide: beyond dim the keys and queries are zero and the decays one, so that the walk below has no condition
    // in it and its LDS reads go out in batches.
    for (int idx0 = lane; idx0 < nr * KD; idx0 += kWave * 8) {
      float kk[8], qq[8], zz[8];
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const int idx = idx0 + b * kWave;
        const int r = idx / KD, d = idx % KD;
        const bool ok = r < nr && d < dim;
        const long at = static_cast<long>(head) * dim + (ok ? d : 0);
        const long row = r0 + (ok ? r : 0);
        kk[b] = load_any(a.k, a.k_dtype, row * a.k_row + at);
        qq[b] = kPass ? load_any(a.q, a.q_dtype, row * a.q_row + at) : 0.f;
        zz[b] = kPerChannel ? load_any(a.z, a.z_dtype, row * a.z_row + at) + (a.z_bias ? a.z_bias[at] : 0.f) : 0.f;
      }
#pragma unroll
      for (int b = 0; b < 8; ++b) {
        const int idx = idx0 + b * kWave;
        const int r = idx / KD, d = idx % KD;
        if (r < nr) {
          const bool ok = d < dim;
          k_s[r][d] = ok ? kk[b] : 0.f;
          if (kPass) q_s[r][d] = ok ? qq[b] * a.q_scale : 0.f;
          if (kPerChannel) a_s[r][d] = ok ? expf(log_sigmoid(zz[b]) * a.inv_tau) : 1.0f;
        }
      }
    }
    float vv[kStage];                  // this thread's column of the stage's values, asked for together
#pragma unroll
    for (int r = 0; r < kStage; ++r)
      vv[r] = (live && r < nr) ? load_any(a.v, a.v_dtype, (r0 + r) * a.v_row + static_cast<long>(head) * vdim + col) : 0.f;
    __syncthreads();
    if (kPass == 0 && blockIdx.x == 0) {
#pragma unroll
      for (int i = 0; i < (KD + kWave - 1) / kWave; ++i) {
        const int d = lane + i * kWave;
        if (d < dim)
          for (int r = 0; r < nr; ++r) prod[i] *= kPerChannel ? a_s[r][d] : decay;
      }
    }
#pragma unroll
    for (int r = 0; r < kStage; ++r) {
      if (r >= nr) break;
      float o = 0.f;
#pragma unroll
      for (int d = 0; d < KD; ++d) {
        S[d] = fmaf(kPerChannel ? a_s[r][d] : decay, S[d], k_s[r][d] * vv[r]);
        if (kPass) o = fmaf(S[d], q_s[r][d], o);
      }
      if (kPass && live) a.out[((r0 + r) * a.heads + head) * vdim + col] = o;
    }
  }
  if (kPass == 0) {
    if (live) {
#pragma unroll
      for (int d = 0; d < KD; ++d)
        if (d < dim) a.chunk_state[chunk_at + static_cast<long>(d) * vdim] = S[d];
    }
    if (blockIdx.x == 0) {
#pragma unroll
      for (int i = 0; i < (KD + kWave - 1) / kWave; ++i) {
        const int d = lane + i * kWave;
        if (d < dim) a.chunk_decay[(chunk_id * a.heads + head) * dim + d] = prod[i];
      }
    }
  } else if (n_chunks < 2 && live) {
#pragma unroll
    for (int d = 0; d < KD; ++d)
      if (d < dim) a.state[slot_at + static_cast<long>(d) * vdim] = S[d];
  }
}

// Between the passes: a thread takes one element (channel d, column c) of one (request, head) with two chunks or more,
// replaces every chunk's sum by the state before the chunk and leaves the state after the last one in the slot.
__global__ void decay_scan_between_kernel(float* __restrict__ state, float* __restrict__ chunk_state,
                                          const float* __restrict__ chunk_decay, const int32_t* __restrict__ seq_start,
                                          const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ chunk_base,
                                          int heads, int dim, int vdim) {
  const int s = blockIdx.z / heads, head = blockIdx.z % heads;
  const int n_chunks = (seq_start[s + 1] - seq_start[s] + kChunk - 1) / kChunk;
  if (n_chunks < 2) return;
  const long per_state = static_cast<long>(dim) * vdim;
  const long e = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x;
  if (e >= per_state) return;
  const int d = static_cast<int>(e / vdim);
  float* slot = state + (static_cast<long>(seq_slots[s]) * heads + head) * per_state + e;
  float st = *slot;
  const long id0 = chunk_base[s];
  for (int c0 = 0; c0 < n_chunks; c0 += 8) {          // (eight chunks' numbers asked for together)
    float add[8], dec[8];
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const bool ok = c0 + b < n_chunks;
      const long id = id0 + (ok ? c0 + b : 0);
      add[b] = ok ? chunk_state[(id * heads + head) * per_state + e] : 0.f;
      dec[b] = ok ? chunk_decay[(id * heads + head) * dim + d] : 1.f;
    }
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      if (c0 + b < n_chunks) {
        chunk_state[((id0 + c0 + b) * heads + head) * per_state + e] = st;
        st = fmaf(dec[b], st, add[b]);
      }
    }
  }
  *slot = st;
}

template <int KD>
void launch_scan(const ScanArgs& a, bool per_channel, bool chunked, dim3 grid, hipStream_t s) {
  if (per_channel) {
    if (chunked) decay_scan_kernel<KD, 0, true><<<grid, kWave, 0, s>>>(a);
  } else {
    if (chunked) decay_scan_kernel<KD, 0, false><<<grid, kWave, 0, s>>>(a);
  }
  if (chunked) {
    const long per_state = static_cast<long>(a.dim) * a.vdim;
    dim3 g2(ceil_div(per_state, 256), 1, grid.z);
    decay_scan_between_kernel<<<g2, 256, 0, s>>>(a.state, a.chunk_state, a.chunk_decay, a.seq_start, a.seq_slots,
                                                 a.chunk_base, a.heads, a.dim, a.vdim);
  }
  if (per_channel) decay_scan_kernel<KD, 1, true><<<grid, kWave, 0, s>>>(a);
  else decay_scan_kernel<KD, 1, false><<<grid, kWave, 0, s>>>(a);
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_rotary_table(const int32_t* positions, const double* freqs, double amp, float* table, int n_rows, int half,
                                 void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && half > 0 && positions && freqs && table, "rotary_table: bad arguments rows=%d half=%d", n_rows, half);
  if (n_rows == 0) return 0;
  const long total = static_cast<long>(n_rows) * half;
  const long g = (total + 255) / 256;
  rotary_table_kernel<<<static_cast<int>(g > 65535 ? 65535 : g), 256, 0, static_cast<hipStream_t>(stream)>>>(
      positions, freqs, amp, table, total, half);
  return check_launch("rotary_table");
}

extern "C" int bc4g_heads_prepare_many(const bc4g_prepare_section* sections, int n_sections, int n_rows, void* stream) {
  BC4G_REQUIRE(sections && n_sections >= 1 && n_sections <= 4 && n_rows >= 0, "heads_prepare: %d sections (1 to 4), %d rows",
               n_sections, n_rows);
  PrepareSections all;
  long heads = 0;
  for (int i = 0; i < n_sections; ++i) {
    const bc4g_prepare_section& p = sections[i];
    BC4G_REQUIRE(p.heads > 0 && p.dim > 0 && p.dim <= kMaxHead && p.half >= 0 && 2 * p.half <= p.dim,
                 "heads_prepare: bad sizes heads=%d dim=%d (at most %d) half=%d", p.heads, p.dim, kMaxHead, p.half);
    BC4G_REQUIRE(p.in && p.out && (p.half == 0 || p.table) && p.in_row >= static_cast<long>(p.heads) * p.dim &&
                 (p.slot_map ? p.page_tokens > 0 : p.out_row >= static_cast<long>(p.heads) * p.dim) &&
                 (p.in_dtype == kF32 || p.in_dtype == kBF16) && (p.out_dtype == kF32 || p.out_dtype == kBF16),
                 "heads_prepare: a tensor is missing, a row is shorter than its heads, or a dtype is unknown");
    all.s[i] = p;
    heads += p.heads;
  }
  all.n = n_sections;
  BC4G_REQUIRE(heads <= 65535, "heads_prepare: %ld heads are beyond the grid limit", heads);
  if (n_rows == 0) return 0;
  dim3 grid(n_rows, static_cast<unsigned>(heads));
  heads_prepare_kernel<<<grid, kWave, 0, static_cast<hipStream_t>(stream)>>>(all);
  return check_launch("heads_prepare");
}

extern "C" int bc4g_heads_prepare(const void* in, int in_dtype, long in_row, const float* bias, const float* norm_w, float eps,
                                  const float* table, int half, float factor, void* out, int out_dtype, long out_row,
                                  const int32_t* slot_map, int page_tokens, long page_stride, long head_stride,
                                  long token_stride, int n_rows, int heads, int dim, void* stream) {
  const bc4g_prepare_section one{in, bias, norm_w, table, out, slot_map, in_row, out_row, page_stride, head_stride, token_stride,
                                 in_dtype, out_dtype, half, page_tokens, heads, dim, eps, factor, 0, 0, 0};
  return bc4g_heads_prepare_many(&one, 1, n_rows, stream);
}

extern "C" int bc4g_heads_finish(const float* o, const float* w, float eps, float factor, const void* gate, int gate_dtype,
                                 long gate_row, int act, void* out, int out_dtype, int n_rows, int heads, int vdim, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && heads > 0 && heads <= 65535 && vdim > 0 && vdim <= kMaxHead,
               "heads_finish: bad sizes rows=%d heads=%d vdim=%d (at most %d)", n_rows, heads, vdim, kMaxHead);
  BC4G_REQUIRE(o && out && act >= 0 && act <= 2 && (!gate || gate_row >= static_cast<long>(heads) * vdim) &&
               (out_dtype == kF32 || out_dtype == kBF16) && (!gate || gate_dtype == kF32 || gate_dtype == kBF16),
               "heads_finish: a tensor is missing, the gate's rows are shorter than the heads, or a dtype is unknown");
  if (n_rows == 0) return 0;
  dim3 grid(n_rows, heads);
  heads_finish_kernel<<<grid, kWave, 0, static_cast<hipStream_t>(stream)>>>(o, w, eps, factor, gate, gate_dtype, gate_row, act,
                                                                           out, out_dtype, heads, vdim);
  return check_launch("heads_finish");
}

extern "C" int bc4g_decay_scan_max_dim() { return 256; }

extern "C" int bc4g_decay_scan(const void* q, int q_dtype, long q_row, float q_scale, const void* k, int k_dtype, long k_row,
                               const void* v, int v_dtype, long v_row, const float* head_decay, const void* z, int z_dtype,
                               long z_row, const float* z_bias, float inv_tau, float* out, float* state, float* chunk_state,
                               float* chunk_decay, const int32_t* seq_start, const int32_t* seq_slots,
                               const int32_t* chunk_base, int n_rows, int n_seqs, int most_rows, int heads, int dim, int vdim,
                               void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_seqs >= 0 && most_rows >= 0 && heads > 0 && dim > 0 && dim <= 256 && vdim > 0,
               "decay_scan: bad sizes T=%d S=%d heads=%d dim=%d (at most 256) vdim=%d", n_rows, n_seqs, heads, dim, vdim);
  BC4G_REQUIRE(static_cast<long>(n_seqs) * heads <= 65535, "decay_scan: %d requests x %d heads are beyond the grid limit", n_seqs, heads);
  BC4G_REQUIRE(q && k && v && out && state && seq_start && seq_slots && (head_decay || z), "decay_scan: a tensor is missing");
  const long hd = static_cast<long>(heads) * dim, hv = static_cast<long>(heads) * vdim;
  BC4G_REQUIRE(q_row >= hd && k_row >= hd && v_row >= hv && (!z || z_row >= hd), "decay_scan: a row is shorter than its heads");
  for (int dt : {q_dtype, k_dtype, v_dtype, z ? z_dtype : 0})
    BC4G_REQUIRE(dt == kF32 || dt == kBF16, "decay_scan: unknown dtype %d", dt);
  if (n_rows == 0 || n_seqs == 0 || most_rows == 0) return 0;
  const int most_chunks = ceil_div(most_rows, kChunk);
  const bool chunked = most_chunks >= 2;
  BC4G_REQUIRE(!chunked || (chunk_state && chunk_decay && chunk_base), "decay_scan: requests of several chunks need scratch memory");
  BC4G_REQUIRE(most_chunks <= 65535, "decay_scan: %d rows of one request are beyond the grid limit", most_rows);
  ScanArgs a{q, q_dtype, q_row, q_scale, k, k_dtype, k_row, v, v_dtype, v_row, head_decay, z, z_dtype, z_row, z_bias, inv_tau,
             out, state, chunk_state, chunk_decay, seq_start, seq_slots, chunk_base, heads, dim, vdim};
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(ceil_div(vdim, kWave), most_chunks, n_seqs * heads);
  const bool per_channel = z != nullptr;
  if (dim <= 16) launch_scan<16>(a, per_channel, chunked, grid, s);
  else if (dim <= 32) launch_scan<32>(a, per_channel, chunked, grid, s);
  else if (dim <= 64) launch_scan<64>(a, per_channel, chunked, grid, s);
  else if (dim <= 128) launch_scan<128>(a, per_channel, chunked, grid, s);
  else launch_scan<256>(a, per_channel, chunked, grid, s);
  return check_launch("decay_scan");
}
