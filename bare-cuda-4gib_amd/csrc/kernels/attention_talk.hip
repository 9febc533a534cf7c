// Windowed softmax attention over a paged cache whose heads' weights are mixed by a matrix before they meet the values
// ("talking heads" after the softmax), with a sink in every head's denominator, a penalty on distance in the scores and
// a gate per head on the output.  Plain float arithmetic on float or bfloat16 caches: scores, weights and sums are float32.
//
//   score_g(p, j) = q_g . k_j * scale - far1_g ln(1 + far2_g (p - j))            for p - window < j <= p
//   w_g(p, j)     = exp(score_g) / (sum over the visible j of exp(score_g) + exp(sink_g))
//   o_h(p)        = sigmoid(gate_h(p)) * sum_j (sum_g talk[h, g] w_g(p, j)) v_j       with the values of h's own key/value head
//
// The mixing needs every head's finished weight at a key, and a weight is finished only when its row's denominator is
// known: so a workgroup is one row with all its heads, and it walks the row's keys twice.  The first walk leaves every
// head's maximum and denominator; the second works the scores out again, turns them into weights in LDS (head x 64 keys),
// mixes them and adds the values up.  A wave owns the heads w, w + waves, ...: their scores, their statistics, their
// outputs.  Where the caller gives room for them (heads x reach floats a row, in memory: LDS could not hold them), the
// first walk leaves its scores there and the second reads them back -- a lane reads what it wrote itself -- instead of
// working the products out again; without that room the second walk computes them once more.
// Caches: keys [page, kv_head, token, dim], values [page, kv_head, token, vdim].
//
// Few rows with long walks (decoding) would leave most of the GPU idle: then a row's keys are cut into parts, a workgroup
// each, and the two walks become two launches -- the first leaves every part's maxima and sums, the second combines
// them into the row's statistics, weighs its own part's values and leaves a partial output (the weights are finished,
// so the parts' outputs simply add up) -- and a third adds the parts and applies the gate.  With kept scores the cut
// goes on through the heads: workgroup z of a part takes the z-th head of every wave (its scores and statistics in
// the first launch, its mixing and its weighted sums in the second, where every head's weights of the tile are made
// from the kept scores by whoever needs them).
#include <float.h>
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kMaxWaves = 8;
constexpr int kMaxHeads = 64;
constexpr int kMaxDim = 256, kMaxVdim = 256;
constexpr int kMaxQ = 8192;      // heads * (dim rounded up to 32): what the queries may take in LDS
constexpr int kAhead = 8;        // keys whose values a lane asks for together

__device__ inline float4 load_four(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ inline float4 load_four(const bf16_t* p) {
  const uint2 bits = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(bits.x << 16), __uint_as_float(bits.x & 0xffff0000u),
                     __uint_as_float(bits.y << 16), __uint_as_float(bits.y & 0xffff0000u));
}

__device__ inline void wave_sync() {      // LDS written by this wave's lanes is read by its other lanes
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// SL: heads a wave owns at most.  E4: for the scores eight lanes share a key, each with 4 E4 of its dimensions
// (dim <= 32 E4).  LPK: lanes that share a key for the weighted sums, each with four neighbouring value dimensions
// (vdim <= 4 LPK); 0: a lane holds dimensions lane, lane + 64, ... (any vdim).
template <typename T, int SL, int E4, int LPK>
__global__ __launch_bounds__(kMaxWaves * kWave) void attention_talk_kernel(
    const float* __restrict__ q, long q_row, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ positions, const float* __restrict__ sink, const float* __restrict__ far1,
    const float* __restrict__ far2, const float* __restrict__ talk, const void* __restrict__ gate, int gate_dtype,
    long gate_row, void* __restrict__ out, int out_dtype, int n_heads, int n_kv_heads, int dim, int vdim, int page_tokens,
    int window, float scale, int n_parts, int phase, float* __restrict__ stats, float* __restrict__ partial,
    float* __restrict__ kept, long kept_stride, int by_slot) {
  // phase 0: both walks over all keys, the finished output.  1: the first walk over this part's keys -> stats
  // [row, part, head, (max, sum)].  2: the second walk over this part's keys with all parts' stats -> partial
  // [row, part, head, vdim].  kept [row, head, kept_stride]: the first walk's scores, by visible key (or null).
  extern __shared__ __align__(16) float dyn[];
  __shared__ long k_at[kMaxWaves][kWave];     // where every key of the tile lies (key/value head 0)
  __shared__ long v_at[kMaxWaves][kWave];
  __shared__ float s_s[kMaxWaves][kWave];     // a head's scores on their way from (key, piece) lanes to lane = key
  __shared__ float m_s[kMaxWaves][kWave];     // a head's mixed weights, lane = key -> every lane
  const int dimp = 32 * E4;                   // a head's queries in LDS, zeros beyond dim
  const int hp = (n_heads + 7) / 8 * 8;       // heads in whole eights: the mixing takes eight at a time
  float* q_s = dyn;                           // [heads][dimp]
  float* p_s = dyn + n_heads * dimp;          // [hp][64]: the tile's weights (zeros beyond the heads)
  float* t_s = p_s + hp * kWave;              // [heads][hp]: the mixing matrix (zeros beyond the heads)
  const int row = blockIdx.x, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n_waves = blockDim.x / kWave;
  const int per_kv = n_heads / n_kv_heads;
  const int pos = positions[row];
  const int32_t* table = block_table + static_cast<long>(row_seq[row]) * table_stride;
  for (int i = threadIdx.x; i < n_heads * dimp; i += blockDim.x) {
    const int h = i / dimp, c = i % dimp;
    q_s[i] = c < dim ? q[row * q_row + static_cast<long>(h) * dim + c] : 0.f;
  }
  for (int i = n_heads * kWave + threadIdx.x; i < hp * kWave; i += blockDim.x) p_s[i] = 0.f;
  if (talk)
    for (int i = threadIdx.x; i < n_heads * hp; i += blockDim.x) t_s[i] = i % hp < n_heads ? talk[(i / hp) * n_heads + i % hp] : 0.f;
  __syncthreads();

  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int total = pos - first + 1;
  const int key_part = blockIdx.y;
  const int only = by_slot ? static_cast<int>(blockIdx.z) : -1;      // the one head of each wave this workgroup serves (-1: all)
  int v_begin = 0, v_end = total;
  if (n_parts > 1) {                          // whole tiles of 64 keys a part; the last parts may be empty
    const int tiles = (total + kWave - 1) / kWave;
    const int per = (tiles + n_parts - 1) / n_parts;
    v_begin = key_part * per * kWave < total ? key_part * per * kWave : total;
    v_end = v_begin + per * kWave < total ? v_begin + per * kWave : total;
  }
  const bool by_four = dim % 4 == 0 && reinterpret_cast<uintptr_t>(k_cache) % (4 * sizeof(T)) == 0;
  const int sub = lane / 8, piece = lane % 8;
  int k_col[E4];
#pragma unroll
  for (int e = 0; e < E4; ++e) {
    const int c = piece * 4 * E4 + 4 * e;
    k_col[e] = c + 4 <= dim ? c : (dim >= 4 ? dim - 4 : 0);
  }
  const long k_head = static_cast<long>(page_tokens) * dim, v_head = static_cast<long>(page_tokens) * vdim;

  // The scores of head h for the wave's tile (k_at filled, synchronized): lane = key.  Lanes without a key compute on
  // the tile's first key; the caller drops them.
  auto scores = [&](int h, int j) -> float {
    const int kvh = h / per_kv;
    float dot;
    if (by_four) {
      float4 q_r[E4];
#pragma unroll
      for (int e = 0; e < E4; ++e) q_r[e] = *reinterpret_cast<const float4*>(&q_s[h * dimp + piece * 4 * E4 + 4 * e]);
#pragma unroll
      for (int it = 0; it < 8; it += 2) {                  // sixteen keys' pieces asked for together
        float4 kk[2][E4];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const T* kp = k_cache + k_at[wave][8 * (it + u) + sub] + kvh * k_head;
#pragma unroll
          for (int e = 0; e < E4; ++e) kk[u][e] = load_four(kp + k_col[e]);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          float part = 0.f;
#pragma unroll
          for (int e = 0; e < E4; ++e) {
            part = fmaf(q_r[e].x, kk[u][e].x, part), part = fmaf(q_r[e].y, kk[u][e].y, part);
            part = fmaf(q_r[e].z, kk[u][e].z, part), part = fmaf(q_r[e].w, kk[u][e].w, part);
          }
          part += __shfl_xor(part, 1, kWave), part += __shfl_xor(part, 2, kWave), part += __shfl_xor(part, 4, kWave);
          if (piece == 0) s_s[wave][8 * (it + u) + sub] = part;
        }
      }
      wave_sync();
      dot = s_s[wave][lane];
      wave_sync();
    } else {
      const T* kp = k_cache + k_at[wave][lane] + kvh * k_head;
      dot = 0.f;
      for (int c = 0; c < dim; ++c) dot = fmaf(q_s[h * dimp + c], to_float(kp[c]), dot);
    }
    float sc = dot * scale;
    if (far1) sc -= far1[h] * log1pf(far2[h] * static_cast<float>(pos - j));
    return sc;
  };
  auto place = [&](int v0, bool& seen, int& j) {      // this lane's key of the tile that begins at visible key v0
    seen = v0 + lane < total;
    j = first + (seen ? v0 + lane : v0);
    const long page = table[j / page_tokens];
    const int off = j % page_tokens;
    k_at[wave][lane] = (page * n_kv_heads * page_tokens + off) * dim;
    v_at[wave][lane] = (page * n_kv_heads * page_tokens + off) * vdim;
    wave_sync();
  };

  // ---- first walk: every head's maximum and denominator --------------------------------------------------------------
  float mx[SL], inv[SL];
#pragma unroll
  for (int s = 0; s < SL; ++s) mx[s] = -INFINITY, inv[s] = 0.f;
  for (int v0 = v_begin; v0 < v_end && phase != 2; v0 += kWave) {
    bool seen;
    int j;
    place(v0, seen, j);
#pragma unroll
    for (int s = 0; s < SL; ++s) {
      const int h = wave + s * n_waves;
      if (h >= n_heads) break;
      if (only >= 0 && s != only) continue;
      float sc = scores(h, j);
      if (kept) kept[(static_cast<long>(row) * n_heads + h) * kept_stride + v0 + lane] = sc;
      if (!seen) sc = -INFINITY;
      const float m_new = fmaxf(mx[s], wave_max(sc));       // finite: the tile's first key is visible
      const float p = seen ? expf(sc - m_new) : 0.f;
      inv[s] = inv[s] * expf(mx[s] - m_new) + wave_sum(p);  // (the sum so far; turned into its inverse below)
      mx[s] = m_new;
    }
    wave_sync();
  }
  if (phase == 1) {                                         // this part's maxima and sums (an empty part: -inf, 0)
#pragma unroll
    for (int s = 0; s < SL; ++s) {
      const int h = wave + s * n_waves;
      if (h >= n_heads) break;
      if (only >= 0 && s != only) continue;
      float* at = stats + ((static_cast<long>(row) * n_parts + key_part) * n_heads + h) * 2;
      if (lane == 0) at[0] = mx[s], at[1] = inv[s];
    }
    return;
  }
  if (phase == 2) {                                         // the row's statistics from every part's (the first is never empty)
#pragma unroll
    for (int s = 0; s < SL; ++s) {
      const int h = wave + s * n_waves;
      if (h >= n_heads) break;
      const float* of = stats + (static_cast<long>(row) * n_parts * n_heads + h) * 2;
      const bool mine = lane < n_parts;                     // a lane a part (at most 64): one trip to memory for all of them
      const float m_i = mine ? of[static_cast<long>(lane) * n_heads * 2] : -INFINITY;
      const float s_i = mine ? of[static_cast<long>(lane) * n_heads * 2 + 1] : 0.f;
      const float top = wave_max(m_i);
      const float sum = wave_sum(m_i > -INFINITY ? s_i * expf(m_i - top) : 0.f);
      mx[s] = top, inv[s] = sum;
    }
  }
#pragma unroll
  for (int s = 0; s < SL; ++s) {
    const int h = wave + s * n_waves;
    if (h >= n_heads) break;
    float sum = inv[s];
    if (sink) {                                            // the sink: a term of the denominator, never scaled
      const float sk = sink[h], top = fmaxf(mx[s], sk);
      sum = fmaf(sum, expf(mx[s] - top), expf(sk - top));
      mx[s] = top;
    }
    inv[s] = 1.0f / sum;
  }

  // ---- second walk: weights, mixed, times values ------------------------------------------------------------------------
  constexpr int VPL = 4;
  constexpr int KPI = LPK ? kWave / LPK : 1;      // keys a load of values brings
  const int vgroup = LPK ? lane / LPK : 0;
  int vcol[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) vcol[i] = LPK ? 4 * (lane % (LPK ? LPK : 1)) + i : lane + i * kWave;
  const int vfrom = LPK ? (vcol[0] + 4 <= vdim ? vcol[0] : vdim - 4) : 0;
  float acc[SL][VPL];
#pragma unroll
  for (int s = 0; s < SL; ++s)
#pragma unroll
    for (int i = 0; i < VPL; ++i) acc[s][i] = 0.f;
  for (int v0 = v_begin; v0 < v_end; v0 += kWave) {
    bool seen;
    int j;
    place(v0, seen, j);
#pragma unroll
    for (int s = 0; s < SL; ++s) {
      const int h = wave + s * n_waves;
      if (h >= n_heads) break;
      const float sc = kept ? kept[(static_cast<long>(row) * n_heads + h) * kept_stride + v0 + lane] : scores(h, j);
      p_s[h * kWave + lane] = seen ? expf(sc - mx[s]) * inv[s] : 0.f;
    }
    __syncthreads();                                        // every head's weights of this tile are there
    const int n_here = total - v0 < kWave ? total - v0 : kWave;
#pragma unroll
    for (int s = 0; s < SL; ++s) {
      const int h = wave + s * n_waves;
      if (h >= n_heads) break;
      if (only >= 0 && s != only) continue;
      float mixed;
      if (talk) {
        mixed = 0.f;
        const float* t_row = t_s + h * hp;
        for (int g0 = 0; g0 < hp; g0 += 8) {             // (eight reads of each kind in flight together)
#pragma unroll
          for (int u = 0; u < 8; ++u) mixed = fmaf(t_row[g0 + u], p_s[(g0 + u) * kWave + lane], mixed);
        }
      } else {
        mixed = p_s[h * kWave + lane];
      }
      m_s[wave][lane] = mixed;
      wave_sync();
      const long v_off = (h / per_kv) * v_head;
      for (int j0 = 0; j0 < n_here; j0 += kAhead * KPI) {  // (keys beyond the tile's last weigh zero and read the first key's values)
        float vv[kAhead][VPL];
#pragma unroll
        for (int b = 0; b < kAhead; ++b) {
          const T* vrow = v_cache + v_at[wave][(j0 + b * KPI + vgroup) % kWave] + v_off;
          if (LPK) {
            const float4 four = load_four(vrow + vfrom);
            vv[b][0] = four.x, vv[b][1] = four.y, vv[b][2] = four.z, vv[b][3] = four.w;
          } else {
#pragma unroll
            for (int i = 0; i < VPL; ++i) vv[b][i] = to_float(vrow[vcol[i] < vdim ? vcol[i] : vdim - 1]);
          }
        }
#pragma unroll
        for (int b = 0; b < kAhead; ++b) {
          const int key = j0 + b * KPI + vgroup;
          const float p = key < kWave ? m_s[wave][key] : 0.f;
#pragma unroll
          for (int i = 0; i < VPL; ++i) acc[s][i] = fmaf(p, vv[b][i], acc[s][i]);
        }
      }
      wave_sync();
    }
    __syncthreads();                                        // before the next tile's weights take their place
  }
  const bool writer = !LPK || lane < LPK;                   // (the other lanes hold copies)
#pragma unroll
  for (int s = 0; s < SL; ++s) {
    const int h = wave + s * n_waves;
    if (h >= n_heads) break;
    if (only >= 0 && s != only) continue;
    float g = 1.0f;
    if (gate) {
      const long at = row * gate_row + h;
      const float z = gate_dtype == kF32 ? static_cast<const float*>(gate)[at] : to_float(static_cast<const bf16_t*>(gate)[at]);
      g = 1.0f / (1.0f + expf(-z));
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      float r = acc[s][i];
      if (LPK && LPK < kWave) {                             // the groups of lanes that took different keys: their sums together
        if (LPK <= 16) r += __shfl_xor(r, 16, kWave);
        r += __shfl_xor(r, 32, kWave);
      }
      const int c = vcol[i];
      if (c >= vdim || !writer) continue;
      if (phase == 2) {
        partial[((static_cast<long>(row) * n_parts + key_part) * n_heads + h) * vdim + c] = r;
        continue;
      }
      const long at = (static_cast<long>(row) * n_heads + h) * vdim + c;
      if (out_dtype == kF32) static_cast<float*>(out)[at] = r * g;
      else static_cast<bf16_t*>(out)[at] = from_float<bf16_t>(r * g);
    }
  }
}

// out[row, h, c] = sigmoid(gate[row, h]) * sum over the parts of partial[row, part, h, c].
__global__ void attention_talk_finish_kernel(const float* __restrict__ partial, int n_parts, const void* __restrict__ gate,
                                             int gate_dtype, long gate_row, void* __restrict__ out, int out_dtype, long n_rows,
                                             int n_heads, int vdim) {
  const long per_row = static_cast<long>(n_heads) * vdim;
  const long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n_rows * per_row) return;
  const long row = i / per_row, rest = i % per_row;
  const int h = static_cast<int>(rest / vdim);
  float r = 0.f;
  for (int p = 0; p < n_parts; ++p) r += partial[(row * n_parts + p) * per_row + rest];
  if (gate) {
    const long at = row * gate_row + h;
    const float z = gate_dtype == kF32 ? static_cast<const float*>(gate)[at] : to_float(static_cast<const bf16_t*>(gate)[at]);
    r *= 1.0f / (1.0f + expf(-z));
  }
  if (out_dtype == kF32) static_cast<float*>(out)[i] = r;
  else static_cast<bf16_t*>(out)[i] = from_float<bf16_t>(r);
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_attention_talk(const float* q, long q_row, const void* k_cache, const void* v_cache, int cache_dtype,
                                   const int32_t* block_table, int table_stride, const int32_t* row_seq,
                                   const int32_t* positions, const float* sink, const float* far1, const float* far2,
                                   const float* talk, const void* gate, int gate_dtype, long gate_row, void* out,
                                   int out_dtype, int n_rows, int n_heads, int n_kv_heads, int dim, int vdim,
                                   int page_tokens, int window, float scale, int n_parts, float* stats, float* partial,
                                   float* kept, long kept_stride, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && n_heads > 0 && n_heads <= kMaxHeads && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
               "attention_talk: bad sizes T=%d heads=%d/%d (at most %d heads)", n_rows, n_heads, n_kv_heads, kMaxHeads);
  BC4G_REQUIRE(dim > 0 && dim <= kMaxDim && vdim > 0 && vdim <= kMaxVdim, "attention_talk: dim=%d (at most %d), vdim=%d (at most %d)",
               dim, kMaxDim, vdim, kMaxVdim);
  const int e4 = dim <= 64 ? 2 : 8;
  BC4G_REQUIRE(n_heads * 32 * e4 <= kMaxQ, "attention_talk: %d heads of %d are more than the %d numbers a row's queries may take",
               n_heads, dim, kMaxQ);
  BC4G_REQUIRE(page_tokens > 0 && table_stride > 0 && window >= 0, "attention_talk: bad cache sizes page_tokens=%d table_stride=%d window=%d",
               page_tokens, table_stride, window);
  BC4G_REQUIRE(q && k_cache && v_cache && block_table && row_seq && positions && out && q_row >= static_cast<long>(n_heads) * dim &&
               (!gate || gate_row >= n_heads) && (out_dtype == kF32 || out_dtype == kBF16) &&
               (!gate || gate_dtype == kF32 || gate_dtype == kBF16) && (far1 == nullptr) == (far2 == nullptr),
               "attention_talk: a tensor is missing, a row is shorter than its heads, or a dtype is unknown");
  BC4G_REQUIRE(n_parts >= 1 && n_parts <= kWave && (n_parts == 1 || (stats && partial)),
               "attention_talk: %d parts of a row's keys need room for their statistics and outputs", n_parts);
  BC4G_REQUIRE(!kept || (kept_stride > 0 && kept_stride % kWave == 0), "attention_talk: the kept scores' rows (%ld) must be whole tiles of %d",
               kept_stride, kWave);
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int waves = n_heads < kMaxWaves ? n_heads : kMaxWaves;
  const int slots = (n_heads + waves - 1) / waves;
  const int by_slot = n_parts > 1 && kept && slots > 1;
  const int hp = (n_heads + 7) / 8 * 8;
  const size_t lds = (static_cast<size_t>(n_heads) * (32 * e4 + hp) + static_cast<size_t>(hp) * kWave) * sizeof(float);
  const bool v_four = vdim % 4 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0;
#define BC4G_TALK_PHASE(T, SL, E, V, PHASE)                                                                                 \
  attention_talk_kernel<T, SL, E, V><<<dim3(n_rows, n_parts, by_slot ? slots : 1), waves * kWave, lds, s>>>(                \
      q, q_row, static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), block_table, table_stride, row_seq, positions, \
      sink, far1, far2, talk, gate, gate_dtype, gate_row, out, out_dtype, n_heads, n_kv_heads, dim, vdim, page_tokens, window, \
      scale, n_parts, PHASE, stats, partial, kept, kept_stride, by_slot)
#define BC4G_TALK(T, SL, E, V)                                                                                              \
  do { if (n_parts == 1) BC4G_TALK_PHASE(T, SL, E, V, 0); else { BC4G_TALK_PHASE(T, SL, E, V, 1); BC4G_TALK_PHASE(T, SL, E, V, 2); } } while (0)
#define BC4G_TALK_V(T, SL, E)                                                                                               \
  do { if (!v_four) BC4G_TALK(T, SL, E, 0); else if (vdim <= 64) BC4G_TALK(T, SL, E, 16); else if (vdim <= 128) BC4G_TALK(T, SL, E, 32); else BC4G_TALK(T, SL, E, 64); } while (0)
#define BC4G_TALK_E(T, SL)                                                                                                  \
  do { if (e4 == 2) BC4G_TALK_V(T, SL, 2); else BC4G_TALK_V(T, SL, 8); } while (0)
#define BC4G_TALK_S(T)                                                                                                      \
  do { if (slots <= 1) BC4G_TALK_E(T, 1); else if (slots <= 2) BC4G_TALK_E(T, 2); else if (slots <= 4) BC4G_TALK_E(T, 4); else BC4G_TALK_E(T, 8); } while (0)
  if (cache_dtype == kF32) BC4G_TALK_S(float);
  else if (cache_dtype == kBF16) BC4G_TALK_S(bf16_t);
  else return fail("attention_talk: unknown dtype %d", cache_dtype);
#undef BC4G_TALK
#undef BC4G_TALK_PHASE
#undef BC4G_TALK_V
#undef BC4G_TALK_E
#undef BC4G_TALK_S
  if (n_parts > 1) {
    const long total = static_cast<long>(n_rows) * n_heads * vdim;
    attention_talk_finish_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, s>>>(
        partial, n_parts, gate, gate_dtype, gate_row, out, out_dtype, n_rows, n_heads, vdim);
  }
  return check_launch("attention_talk");
}
