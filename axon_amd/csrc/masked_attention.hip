// Grouped-query attention with the variations a configuration may ask for, each a parameter:
//   * one or two score maps a head (two: differential attention, o = rms(a_1 - lambda a_2) c over one
//     set of values), keys of `dim` and values of `vdim` elements, `heads` query heads over `kv_heads`;
//   * a per-head RMS norm of queries and keys with a gain, rotation of the leading dims in either
//     pairing (places (2i, 2i + 1) or (i, i + n / 2)) with cos and sin scaled by a factor;
//   * what a position sees: every earlier position, the last `size` positions (a sliding window), or
//     the earlier positions of its own chunk of `size` (chunks counted from position 0);
//   * scores bent by cap tanh(s / cap);
//   * an elementwise gate sigmoid(g) on the concatenated heads.
//
// A page of the cache holds, for its positions, the key rows [page_size][kv_heads maps dim] and behind
// them the values with the positions of one dim side by side, [kv_heads vdim][page_size] (the operand
// layout of the matrix cores' weighted sum).  Scores, weights, sums and norms are 32-bit in both builds.
#include <math.h>

#include "api.h"
#include "common.h"

namespace {

enum { MASK_CAUSAL = 0, MASK_WINDOW = 1, MASK_CHUNK = 2 };

__device__ inline int first_seen(int pos, int mask_kind, int mask_size) {
  if (mask_kind == MASK_WINDOW) return max(0, pos + 1 - mask_size);
  if (mask_kind == MASK_CHUNK) return pos / mask_size * mask_size;
  return 0;
}

// One block per token, a wave a unit (one map of one head) at a time.  proj [T, stride] float32 holds
// the projections' results: n_q units of `dim` from q_at, n_k units from k_at, and v_width values from
// v_at (v_at may equal k_at: the values are the keys as projected).  Units are RMS-normed with a gain
// shared by all units (if given), their first rot dims rotated by the step's table [T, rot / 2, 2]
// (sin, cos), and stored: queries into q_out [T, n_q dim], keys and values into the token's page.
__global__ void __launch_bounds__(256)
heads_prepare_kernel(const float* __restrict__ proj, long stride, int q_at, int n_q, int k_at, int n_k, int v_at, int v_width,
                     int dim, const void* __restrict__ q_gain, int q_gain_is_f32, const void* __restrict__ k_gain,
                     int k_gain_is_f32, float eps, int rot, int neighbours, float magnitude, const float* __restrict__ table,
                     const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                     const int32_t* __restrict__ block_table, int table_stride, elem_t* __restrict__ cache, int page_size,
                     elem_t* __restrict__ q_out, int write_kv) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* row = proj + (long)t * stride;
  const int half = rot / 2;
  const float* tab = table + (long)t * half * 2;
  const int kw = n_k * dim;
  elem_t* page_base = nullptr;
  int in_page = 0;
  if (write_kv) {
    const int pos = positions[t];
    const int page = block_table[(long)seq_rows[t] * table_stride + pos / page_size];
    page_base = cache + (long)page * page_size * (kw + v_width);
    in_page = pos % page_size;
  }
  const int n_units = n_q + (write_kv ? n_k : 0);
  for (int u = wave; u < n_units; u += 4) {
    const bool is_q = u < n_q;
    const float* src = row + (is_q ? q_at + u * dim : k_at + (u - n_q) * dim);
    elem_t* dst = is_q ? q_out + ((long)t * n_q + u) * dim : page_base + (long)in_page * kw + (long)(u - n_q) * dim;
    const void* gain = is_q ? q_gain : k_gain;
    const int gain_is_f32 = is_q ? q_gain_is_f32 : k_gain_is_f32;
    float inv = 1.0f;
    if (gain != nullptr) {
      float ss = 0.0f;
      for (int i = lane; i < dim; i += 64) ss = fmaf(src[i], src[i], ss);
      inv = 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps);
    }
    for (int i = lane; i < half; i += 64) {
      const int ia = neighbours ? 2 * i : i, ib = neighbours ? 2 * i + 1 : i + half;
      float a = src[ia], b = src[ib];
      if (gain != nullptr) {
        a = (a * inv) * load_vec(gain, gain_is_f32, ia);
        b = (b * inv) * load_vec(gain, gain_is_f32, ib);
      }
      const float s = tab[2 * i] * magnitude, c = tab[2 * i + 1] * magnitude;
      dst[ia] = from_float(__fsub_rn(__fmul_rn(a, c), __fmul_rn(b, s)));
      dst[ib] = from_float(__fadd_rn(__fmul_rn(b, c), __fmul_rn(a, s)));
    }
    for (int i = rot + lane; i < dim; i += 64) {
      float a = src[i];
      if (gain != nullptr) a = (a * inv) * load_vec(gain, gain_is_f32, i);
      dst[i] = from_float(a);
    }
  }
  if (!write_kv) return;
  elem_t* by_dim = page_base + (long)page_size * kw + in_page;
  for (int i = threadIdx.x; i < v_width; i += 256) by_dim[(long)i * page_size] = from_float(row[v_at + i]);
}

// One wave per (token, head), four waves a block; any sizes, both builds.  For each map: positions
// first ..= pos in blocks of 64 aligned to absolute position, ascending; lane j scores position
// 64 b + j against the query in LDS, the block's maximum and sum are butterflies, and the running
// (m, l, o) are rescaled block by block; lane d owns value dims d, d + 64, ...  Then the maps are
// combined, normed and gated, and the head's vdim outputs stored.
#define MA_WAVES 4
#define MA_OWN 4      // value dims a lane owns: vdim up to 256
__global__ void __launch_bounds__(MA_WAVES * 64)
masked_attention_kernel(const elem_t* __restrict__ q, const elem_t* __restrict__ cache, const int32_t* __restrict__ block_table,
                        int table_stride, const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                        const float* __restrict__ gate, long gate_stride, elem_t* __restrict__ out, int n_tokens, int heads,
                        int kv_heads, int maps, int dim, int vdim, int page_size, int mask_kind, int mask_size, float scale,
                        float softcap, float lambda, float out_scale, float eps) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long item = (long)blockIdx.x * MA_WAVES + wave;
  const bool active = item < (long)n_tokens * heads;
  const int t = active ? (int)(item / heads) : 0, h = active ? (int)(item % heads) : 0;
  const int qw = maps * dim;
  float* qs = smem + (long)wave * qw;
  const elem_t* qsrc = q + ((long)t * heads + h) * qw;
  if (active)
    for (int i = lane; i < qw; i += 64) qs[i] = to_float(qsrc[i]);
  __syncthreads();
  if (!active) return;
  const int g = h / (heads / kv_heads);
  const int kw = kv_heads * maps * dim;
  const long page_elems = (long)page_size * (kw + kv_heads * vdim);
  const int pos = positions[t];
  const int lo = first_seen(pos, mask_kind, mask_size);
  const int32_t* pages = block_table + (long)seq_rows[t] * table_stride;
  float o[MA_OWN];
#pragma unroll
  for (int i = 0; i < MA_OWN; ++i) o[i] = 0.0f;
  for (int mp = 0; mp < maps; ++mp) {
    float acc[MA_OWN];
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) acc[i] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    const float* qm = qs + mp * dim;
    for (int b = lo / 64; b <= pos / 64; ++b) {
      const int p = b * 64 + lane;
      const bool seen = p >= lo && p <= pos;
      float s = -INFINITY;
      if (seen) {
        const elem_t* key = cache + (long)pages[p / page_size] * page_elems + (long)(p % page_size) * kw + (g * maps + mp) * dim;
        float dot = 0.0f;
        for (int i = 0; i < dim; ++i) dot = fmaf(qm[i], to_float(key[i]), dot);
        s = dot * scale;
        if (softcap > 0.0f) s = softcap * tanhf(s / softcap);
      }
      const float m_new = fmaxf(m, wave_max(s));
      const float w = seen ? expf(s - m_new) : 0.0f;
      const float fold = expf(m - m_new);            // 0 at the first block (m = -inf)
      l = fmaf(l, fold, wave_sum(w));
      m = m_new;
#pragma unroll
      for (int i = 0; i < MA_OWN; ++i) acc[i] *= fold;
      const int j_lo = max(lo, b * 64) - b * 64, j_hi = min(pos, b * 64 + 63) - b * 64;
      for (int j = j_lo; j <= j_hi; ++j) {
        const float wj = __shfl(w, j, 64);
        const int pj = b * 64 + j;
        const elem_t* val = cache + (long)pages[pj / page_size] * page_elems + (long)page_size * kw +
                            (long)g * vdim * page_size + pj % page_size;
#pragma unroll
        for (int i = 0; i < MA_OWN; ++i) {
          const int d = lane + 64 * i;
          if (d < vdim) acc[i] = fmaf(wj, to_float(val[(long)d * page_size]), acc[i]);
        }
      }
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) o[i] = mp == 0 ? acc[i] * inv : o[i] - lambda * (acc[i] * inv);
  }
  if (maps > 1) {
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) ss = fmaf(o[i], o[i], ss);     // dims beyond vdim hold 0
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)vdim + eps);
#pragma unroll
    for (int i = 0; i < MA_OWN; ++i) o[i] = (o[i] * inv) * out_scale;
  }
  elem_t* dst = out + ((long)t * heads + h) * vdim;
#pragma unroll
  for (int i = 0; i < MA_OWN; ++i) {
    const int d = lane + 64 * i;
    if (d >= vdim) continue;
    float v = o[i];
    if (gate != nullptr) v *= 1.0f / (1.0f + expf(-gate[(long)t * gate_stride + (long)h * vdim + d]));
    dst[d] = from_float(v);
  }
}

}  // namespace

extern "C" int axk_heads_prepare(const float* proj, long stride, int q_at, int n_q, int k_at, int n_k, int v_at, int v_width,
                                 int dim, const void* q_gain, int q_gain_is_f32, const void* k_gain, int k_gain_is_f32, float eps,
                                 int rot, int neighbours, float magnitude, const float* table, const int32_t* positions,
                                 const int32_t* seq_rows, const int32_t* block_table, int table_stride, void* cache, int page_size,
                                 void* q_out, int n_tokens, int write_kv, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_q > 0 && n_k > 0 && dim > 0 && v_width > 0 && page_size > 0,
              "heads_prepare: bad sizes T=%d q units=%d k units=%d dim=%d values=%d page=%d", n_tokens, n_q, n_k, dim, v_width,
              page_size);
  AXK_REQUIRE(rot >= 0 && rot <= dim && rot % 2 == 0, "heads_prepare: %d rotated dims of %d", rot, dim);
  AXK_REQUIRE(q_at >= 0 && k_at >= 0 && v_at >= 0 && q_at + (long)n_q * dim <= stride && k_at + (long)n_k * dim <= stride &&
              v_at + (long)v_width <= stride, "heads_prepare: the parts do not fit rows of %ld", stride);
  if (n_tokens == 0) return 0;
  heads_prepare_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(
      proj, stride, q_at, n_q, k_at, n_k, v_at, v_width, dim, q_gain, q_gain_is_f32, k_gain, k_gain_is_f32, eps, rot, neighbours,
      magnitude, table, positions, seq_rows, block_table, table_stride, (elem_t*)cache, page_size, (elem_t*)q_out, write_kv);
  AXK_LAUNCH_CHECK("heads_prepare");
  return 0;
}

// 1 where axk_masked_attention runs on the matrix cores.
extern "C" int axk_masked_attention_uses_mfma(int heads, int kv_heads, int maps, int dim, int vdim, int page_size) {
  return 0;
}

extern "C" int axk_masked_attention(const void* q, const void* cache, const int32_t* block_table, int table_stride,
                                    const int32_t* positions, const int32_t* seq_rows, const float* gate, long gate_stride,
                                    void* out, int n_tokens, int heads, int kv_heads, int maps, int dim, int vdim, int page_size,
                                    int mask_kind, int mask_size, float scale, float softcap, float lambda, float out_scale,
                                    float eps, const int32_t* tiles, int n_tiles, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 && page_size > 0,
              "masked_attention: bad sizes T=%d heads=%d kv heads=%d dim=%d vdim=%d page=%d", n_tokens, heads, kv_heads, dim, vdim,
              page_size);
  AXK_REQUIRE(maps == 1 || maps == 2, "masked_attention: %d score maps a head (1 or 2)", maps);
  AXK_REQUIRE(vdim <= 64 * MA_OWN, "masked_attention: values of %d dims (at most %d)", vdim, 64 * MA_OWN);
  AXK_REQUIRE(mask_kind == MASK_CAUSAL || ((mask_kind == MASK_WINDOW || mask_kind == MASK_CHUNK) && mask_size > 0),
              "masked_attention: mask kind %d of size %d", mask_kind, mask_size);
  AXK_REQUIRE((long)maps * dim * MA_WAVES * 4 <= 64 * 1024, "masked_attention: queries of %d dims do not fit LDS", maps * dim);
  if (n_tokens == 0) return 0;
  const long items = (long)n_tokens * heads;
  const size_t lds = (size_t)maps * dim * MA_WAVES * sizeof(float);
  masked_attention_kernel<<<(unsigned)((items + MA_WAVES - 1) / MA_WAVES), MA_WAVES * 64, lds, (hipStream_t)stream>>>(
      (const elem_t*)q, (const elem_t*)cache, block_table, table_stride, positions, seq_rows, gate, gate_stride, (elem_t*)out,
      n_tokens, heads, kv_heads, maps, dim, vdim, page_size, mask_kind, mask_size, scale, softcap, lambda, out_scale, eps);
  AXK_LAUNCH_CHECK("masked_attention");
  return 0;
}
