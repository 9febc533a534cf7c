// Softmax attention over a paged cache whose query heads carry one or two score maps over the same values
// (differential attention: o = a1 - lambda a2), with a window of the last keys plus the first few keys of the
// sequence, keys and values of different sizes, and the head's output optionally divided by its root mean square,
// scaled and gated.  Two further options, each a vector with one number a query head: a sink -- exp(sink) joins the
// softmax's denominator, with no key and no value, never scaled -- and a penalty on distance, r1 ln(1 + r2 (p - j)),
// taken off the scaled score.  Plain float arithmetic on float or bfloat16 caches: scores, weights and sums are float32.
// Three more, for the whole call: a mask by blocks instead of the window (a row sees the keys of its own block of
// `block` positions counted from 0, up to itself), a cap on the scaled score, cap tanh(score / cap), and weights that are no
// softmax: sigmoid(score + point[head]) for every visible key by itself, no maximum, no denominator, no sink.
//
// A row at position p sees key j if j <= p and (window == 0 or p - j < window or j < keep_first); kept keys keep their
// own positions (they were rotated when they were written).  One workgroup per (row, query head): the visible keys --
// the kept first keys, then the window -- are walked in tiles of 64, the workgroup's waves taking the tiles in turn, each
// with a running maximum and sum per map (lane = key for the scores, lane = value dimension for the sums, a tile's
// values read once for both maps); the waves' parts are merged in wave order.  How many waves share a row is the
// caller's choice (few rows over long contexts: many); it changes the order of the sums and nothing else.
// Pages that hold no visible key are never touched.
//
// Caches: keys [page, kv_head * maps + map, token, dim], values [page, kv_head, token, vdim].
#include <float.h>
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kMaxDim = 256;     // of a map's queries and keys
constexpr int kMaxVdim = 256;    // of a head's values

__device__ inline float4 load_four(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ inline float4 load_four(const bf16_t* p) {
  const uint2 bits = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(bits.x << 16), __uint_as_float(bits.x & 0xffff0000u),
                     __uint_as_float(bits.y << 16), __uint_as_float(bits.y & 0xffff0000u));
}

__device__ inline float gate_of(const void* gate, int dtype, long idx, int act) {
  const float z = dtype == kF32 ? static_cast<const float*>(gate)[idx] : to_float(static_cast<const bf16_t*>(gate)[idx]);
  return act == 1 ? z / (1.0f + expf(-z)) : 1.0f / (1.0f + expf(-z));
}

__device__ inline void wave_sync() {      // LDS written by this wave's lanes is read by its other lanes
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int kMaxWaves = 8;     // waves of a workgroup that cut one row's keys among them
constexpr int kAhead = 8;        // keys whose values a lane asks for together

// A workgroup is one (row, query head); its NW waves take the tiles of 64 visible keys in turn (wave w the tiles w,
// w + NW, ...), each with a running maximum and sum per map, and the waves' parts are merged in wave order at the end.
// kNW: the most waves a workgroup may have (it sizes the waves' LDS).  LPK: lanes that share a key for the weighted sums, each
// with four neighbouring value dimensions (vdim <= 4 LPK; 16, 32 or 64), so that a load brings 64 / LPK keys' values in
// pieces of four and the groups' sums are added across lanes at the end; 0: a lane holds dimensions lane, lane + 64, ...
// one key a load (any vdim).
// E4: for the scores, eight lanes share a key and each takes 4 E4 of its dimensions (dim <= 32 E4), so that a load's lanes
// read eight keys' rows end to end -- with a key to a lane every load touched 64 cache lines, and the kernel was as long as
// the CU's one path to memory took to serve them.
template <typename T, int MAPS, int kNW, int LPK, int E4>
__global__ __launch_bounds__(kNW * kWave) void attention_maps_kernel(
    const float* __restrict__ q, long q_row, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ positions, float lambda, int normalize, float eps, float factor,
    const void* __restrict__ gate, int gate_dtype, long gate_row, int gate_act, void* __restrict__ out, int out_dtype,
    int n_heads, int n_kv_heads, int dim, int vdim, int page_tokens, int window, int keep_first, float scale,
    const float* __restrict__ sink, const float* __restrict__ far1, const float* __restrict__ far2, int block, float cap,
    const float* __restrict__ point) {
  __shared__ __align__(16) float q_s[MAPS][kMaxDim];
  __shared__ float p_s[kNW][MAPS][kWave];
  __shared__ long v_at[kNW][kWave];           // where every key of the wave's tile has its values
  __shared__ long k_at[kNW][kWave];           // ... and its first map's dimensions
  __shared__ float s_s[kNW][MAPS][kWave];     // the tile's scores on their way from (key, piece) lanes to lane = key
  __shared__ float part_acc[kNW > 1 ? kNW : 1][MAPS][kNW > 1 ? kMaxVdim : 1];
  __shared__ float part_ml[kNW][MAPS][2];
  const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n_waves = blockDim.x / kWave;
  const int kvh = head / (n_heads / n_kv_heads);
  const int pos = positions[row];
  const int32_t* table = block_table + static_cast<long>(row_seq[row]) * table_stride;
  for (int m = 0; m < MAPS; ++m)      // (zeros beyond dim: the products below run in whole batches)
    for (int c = threadIdx.x; c < kMaxDim; c += blockDim.x)
      q_s[m][c] = c < dim ? q[row * q_row + (static_cast<long>(head) * MAPS + m) * dim + c] : 0.f;
  __syncthreads();

  const int first = block > 0 ? pos - pos % block : (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const float lift = point ? point[head] : 0.f;
  const int kept = window > 0 ? (keep_first < first ? keep_first : first) : 0;      // kept keys before the window
  const int total = kept + (pos - first + 1);
  const float pen1 = far1 ? far1[head] : 0.f, pen2 = far1 ? far2[head] : 0.f;
  const bool by_four = dim % 4 == 0 && reinterpret_cast<uintptr_t>(k_cache) % (4 * sizeof(T)) == 0;
  constexpr int VPL = 4;                // value dimensions a lane holds
  constexpr int KPI = LPK ? kWave / LPK : 1;      // keys a load of values brings
  const int vgroup = LPK ? lane / LPK : 0;
  float mx[MAPS], sum[MAPS], acc[MAPS][VPL];
#pragma unroll
  for (int m = 0; m < MAPS; ++m) {
    mx[m] = -INFINITY, sum[m] = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; ++i) acc[m][i] = 0.f;
  }
  int vcol[VPL];                        // this lane's value dimensions (what lies beyond vdim is dropped at the end)
#pragma unroll
  for (int i = 0; i < VPL; ++i) vcol[i] = LPK ? 4 * (lane % (LPK ? LPK : 1)) + i : lane + i * kWave;
  const int vfrom = LPK ? (vcol[0] + 4 <= vdim ? vcol[0] : vdim - 4) : 0;      // where this lane's piece of four is read (clamped)
  const int sub = lane / 8, piece = lane % 8;          // for the scores: which of a load's eight keys, which piece of its dimensions
  float4 q_r[MAPS][E4];                                 // this lane's piece of the queries (zero beyond dim)
  int k_col[E4];                                        // ... and where it lies in a key's row (clamped)
#pragma unroll
  for (int e = 0; e < E4; ++e) {
    const int c = piece * 4 * E4 + 4 * e;
    k_col[e] = c + 4 <= dim ? c : (dim >= 4 ? dim - 4 : 0);
#pragma unroll
    for (int m = 0; m < MAPS; ++m) q_r[m][e] = *reinterpret_cast<const float4*>(&q_s[m][c]);
  }
  // Nothing in a tile's walk is under a condition: lanes without a key compute on the tile's first key and are dropped
  // by selects, so that loads and LDS reads go out in batches.
  for (int v0 = wave * kWave; v0 < total; v0 += n_waves * kWave) {
    const bool seen = v0 + lane < total;
    const int vi = seen ? v0 + lane : v0;
    const int j = vi < kept ? vi : first + (vi - kept);
    const long page = table[j / page_tokens];
    const int off = j % page_tokens;
    v_at[wave][lane] = ((page * n_kv_heads + kvh) * page_tokens + off) * vdim;
    if (by_four) {
      k_at[wave][lane] = ((page * (n_kv_heads * MAPS) + kvh * MAPS) * page_tokens + off) * dim;
      wave_sync();
#pragma unroll
      for (int it = 0; it < 8; it += 2) {                  // sixteen keys' pieces asked for together
        float4 kk[2][MAPS][E4];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const T* kp = k_cache + k_at[wave][8 * (it + u) + sub];
#pragma unroll
          for (int m = 0; m < MAPS; ++m)
#pragma unroll
            for (int e = 0; e < E4; ++e) kk[u][m][e] = load_four(kp + static_cast<long>(m) * page_tokens * dim + k_col[e]);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int m = 0; m < MAPS; ++m) {
            float part = 0.f;
#pragma unroll
            for (int e = 0; e < E4; ++e) {
              part = fmaf(q_r[m][e].x, kk[u][m][e].x, part), part = fmaf(q_r[m][e].y, kk[u][m][e].y, part);
              part = fmaf(q_r[m][e].z, kk[u][m][e].z, part), part = fmaf(q_r[m][e].w, kk[u][m][e].w, part);
            }
            part += __shfl_xor(part, 1, kWave), part += __shfl_xor(part, 2, kWave), part += __shfl_xor(part, 4, kWave);
            if (piece == 0) s_s[wave][m][8 * (it + u) + sub] = part;
          }
      }
      wave_sync();
    }
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      float dot = 0.f;
      if (by_four) {
        dot = s_s[wave][m][lane];
      } else {
        const T* kp = k_cache + ((page * (n_kv_heads * MAPS) + kvh * MAPS + m) * page_tokens + off) * dim;
        for (int c = 0; c < dim; ++c) dot = fmaf(q_s[m][c], to_float(kp[c]), dot);
      }
      float sc = dot * scale;
      if (far1) sc -= pen1 * log1pf(pen2 * static_cast<float>(pos - j));
      if (cap > 0.f) sc = cap * tanhf(sc / cap);
      if (point) {                                           // a weight a key by itself: nothing to keep up with
        p_s[wave][m][lane] = seen ? 1.0f / (1.0f + expf(-(sc + lift))) : 0.f;
        mx[m] = 0.f;
        continue;
      }
      if (!seen) sc = -INFINITY;
      const float m_new = fmaxf(mx[m], wave_max(sc));       // finite: the tile's first key is visible
      const float p = seen ? expf(sc - m_new) : 0.f;
      const float alpha = expf(mx[m] - m_new);               // 0 on the wave's first tile
      sum[m] = sum[m] * alpha + wave_sum(p);
      mx[m] = m_new;
      p_s[wave][m][lane] = p;
#pragma unroll
      for (int i = 0; i < VPL; ++i) acc[m][i] *= alpha;
    }
    wave_sync();
    const int n_here = total - v0 < kWave ? total - v0 : kWave;
    // (keys beyond the tile's last weigh zero and read the first key's values)
    for (int j0 = 0; j0 < n_here; j0 += kAhead * KPI) {    // kAhead loads asked for together
      float vv[kAhead][VPL];
#pragma unroll
      for (int b = 0; b < kAhead; ++b) {
        const T* vrow = v_cache + v_at[wave][j0 + b * KPI + vgroup];
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
#pragma unroll
        for (int m = 0; m < MAPS; ++m) {
          const float p = p_s[wave][m][j0 + b * KPI + vgroup];
#pragma unroll
          for (int i = 0; i < VPL; ++i) acc[m][i] = fmaf(p, vv[b][i], acc[m][i]);
        }
      }
    }
    wave_sync();
  }
  if (LPK && LPK < kWave) {                              // the groups of lanes that took different keys: their sums together
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
      for (int i = 0; i < VPL; ++i) {
        if (LPK <= 16) acc[m][i] += __shfl_xor(acc[m][i], 16, kWave);
        acc[m][i] += __shfl_xor(acc[m][i], 32, kWave);
      }
  }
  const bool writer = !LPK || lane < LPK;                // (the other lanes hold copies)
  if (kNW > 1 && n_waves > 1) {                          // the waves' parts, merged in wave order
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      if (lane == 0) part_ml[wave][m][0] = mx[m], part_ml[wave][m][1] = sum[m];
#pragma unroll
      for (int i = 0; i < VPL; ++i)
        if (writer) part_acc[wave][m][vcol[i]] = acc[m][i];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      float top = -INFINITY;
      for (int w = 0; w < n_waves; ++w) top = fmaxf(top, part_ml[w][m][0]);
      sum[m] = 0.f;
#pragma unroll
      for (int i = 0; i < VPL; ++i) acc[m][i] = 0.f;
      for (int w = 0; w < n_waves; ++w) {
        const float f = expf(part_ml[w][m][0] - top);    // 0 for a wave that had no tile
        sum[m] = fmaf(part_ml[w][m][1], f, sum[m]);
#pragma unroll
        for (int i = 0; i < VPL; ++i) acc[m][i] = fmaf(part_acc[w][m][vcol[i]], f, acc[m][i]);
      }
      mx[m] = top;                                       // (what the merged sums are counted from)
    }
  }
  if (point) {                                           // (the parts' weights are finished: they were added up as they are)
#pragma unroll
    for (int m = 0; m < MAPS; ++m) sum[m] = 1.0f;
  }
  if (sink && !point) {                                  // the sink: a term of the denominator, with no value
    const float sk = sink[head];
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      const float top = fmaxf(mx[m], sk), f = expf(mx[m] - top);
      sum[m] = fmaf(sum[m], f, expf(sk - top));
#pragma unroll
      for (int i = 0; i < VPL; ++i) acc[m][i] *= f;
    }
  }
  float o[VPL];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    o[i] = acc[0][i] / sum[0];
    if (MAPS == 2) o[i] -= lambda * (acc[MAPS - 1][i] / sum[MAPS - 1]);
    if (vcol[i] >= vdim || !writer) o[i] = 0.f;      // (a lane beyond vdim walked a clamped column; copies count once)
    ss = fmaf(o[i], o[i], ss);
  }
  const float mult = normalize ? factor / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps) : factor;
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int c = vcol[i];
    if (c >= vdim || !writer) continue;
    float r = o[i] * mult;
    if (gate) r *= gate_of(gate, gate_dtype, row * gate_row + static_cast<long>(head) * vdim + c, gate_act);
    const long at = (static_cast<long>(row) * n_heads + head) * vdim + c;
    if (out_dtype == kF32) static_cast<float*>(out)[at] = r;
    else static_cast<bf16_t*>(out)[at] = from_float<bf16_t>(r);
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_attention_maps(const float* q, long q_row, const void* k_cache, const void* v_cache, int cache_dtype,
                                   const int32_t* block_table, int table_stride, const int32_t* row_seq,
                                   const int32_t* positions, float lambda, int normalize, float eps, float factor,
                                   const void* gate, int gate_dtype, long gate_row, int gate_act, void* out, int out_dtype,
                                   int n_rows, int n_heads, int n_kv_heads, int maps, int dim, int vdim, int page_tokens,
                                   int window, int keep_first, float scale, int waves, const float* sink,
                                   const float* far1, const float* far2, int block, float cap, const float* point,
                                   void* stream) {
  BC4G_REQUIRE(waves >= 1 && waves <= kMaxWaves, "attention_maps: %d waves a row (1 to %d)", waves, kMaxWaves);
  BC4G_REQUIRE(n_rows >= 0 && n_heads > 0 && n_heads <= 65535 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
               "attention_maps: bad sizes T=%d heads=%d/%d", n_rows, n_heads, n_kv_heads);
  BC4G_REQUIRE((maps == 1 || maps == 2) && dim > 0 && dim <= kMaxDim && vdim > 0 && vdim <= kMaxVdim,
               "attention_maps: maps=%d (1 or 2), dim=%d (at most %d), vdim=%d (at most %d)", maps, dim, kMaxDim, vdim, kMaxVdim);
  BC4G_REQUIRE(page_tokens > 0 && table_stride > 0 && window >= 0 && keep_first >= 0,
               "attention_maps: bad cache sizes page_tokens=%d table_stride=%d window=%d keep_first=%d", page_tokens,
               table_stride, window, keep_first);
  BC4G_REQUIRE(q && k_cache && v_cache && block_table && row_seq && positions && out &&
               q_row >= static_cast<long>(n_heads) * maps * dim && (!gate || gate_row >= static_cast<long>(n_heads) * vdim) &&
               (gate_act == 1 || gate_act == 2 || !gate) && (out_dtype == kF32 || out_dtype == kBF16) &&
               (!gate || gate_dtype == kF32 || gate_dtype == kBF16),
               "attention_maps: a tensor is missing, a row is shorter than its heads, or a dtype is unknown");
  BC4G_REQUIRE((far1 == nullptr) == (far2 == nullptr), "attention_maps: the distance penalty needs both of its vectors");
  BC4G_REQUIRE(block >= 0 && (block == 0 || (window == 0 && keep_first == 0)) && cap >= 0.f && !(point && sink),
               "attention_maps: block=%d beside window=%d, keep_first=%d; cap=%g; weights without a softmax have no sink", block,
               window, keep_first, static_cast<double>(cap));
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(n_rows, n_heads);
  const bool v_four = vdim % 4 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0;
#define BC4G_MAPS(T, M)                                                                                                   \
  do { if (waves == 1) BC4G_MAPS_V(T, M, 1); else BC4G_MAPS_V(T, M, kMaxWaves); } while (0)
#define BC4G_MAPS_V(T, M, W)                                                                                              \
  do { if (!v_four) BC4G_MAPS_W(T, M, W, 0); else if (vdim <= 64) BC4G_MAPS_W(T, M, W, 16); else if (vdim <= 128) BC4G_MAPS_W(T, M, W, 32); else BC4G_MAPS_W(T, M, W, 64); } while (0)
#define BC4G_MAPS_W(T, M, W, V)                                                                                           \
  do { if (dim <= 64) BC4G_MAPS_E(T, M, W, V, 2); else BC4G_MAPS_E(T, M, W, V, 8); } while (0)
#define BC4G_MAPS_E(T, M, W, V, E)                                                                                        \
  attention_maps_kernel<T, M, W, V, E><<<grid, waves * kWave, 0, s>>>(q, q_row, static_cast<const T*>(k_cache), static_cast<const T*>(v_cache), \
                                                     block_table, table_stride, row_seq, positions, lambda, normalize, eps, \
                                                     factor, gate, gate_dtype, gate_row, gate_act, out, out_dtype, n_heads,  \
                                                     n_kv_heads, dim, vdim, page_tokens, window, keep_first, scale, sink, far1, far2, block, cap, point)
  if (cache_dtype == kF32) {
    if (maps == 1) BC4G_MAPS(float, 1); else BC4G_MAPS(float, 2);
  } else if (cache_dtype == kBF16) {
    if (maps == 1) BC4G_MAPS(bf16_t, 1); else BC4G_MAPS(bf16_t, 2);
  } else {
    return fail("attention_maps: unknown dtype %d", cache_dtype);
  }
#undef BC4G_MAPS
#undef BC4G_MAPS_W
#undef BC4G_MAPS_V
#undef BC4G_MAPS_E
  return check_launch("attention_maps");
}
