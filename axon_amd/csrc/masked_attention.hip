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

#if AXON_BF16
typedef __attribute__((ext_vector_type(8))) __bf16 ma_bf16x8;
typedef __attribute__((ext_vector_type(4))) float ma_f32x4;
__device__ inline ma_bf16x8 ma_frag(uint4 v) { return __builtin_bit_cast(ma_bf16x8, v); }

// The same attention on the matrix cores: one wave per tile of up to sixteen columns, a block of 64
// positions at a time.  A tile of several tokens (consecutive positions of one request) is those
// tokens for one query head; a tile of one token is that token for up to sixteen query heads of
// one key/value head.  Either way all columns read the same keys and values:
//   S^T [position, column] = K [position, dims] Q^T          (dims in chunks of 32, zero-padded),
//   per column a mask of its own, the bend, a maximum, weights and their sum (a lane holds 16
//   positions of its column; the four lanes of a column meet by lane permutation), the running
//   (m, l) and O^T rescaled, then
//   O^T [dim, column] += V^T [dim, position] P^T             (positions in two chunks of 32),
// with K rows and the rows of V^T straight from the page into the first operand (16 or 8 bytes a lane)
// and the rounded weights, as they lie in the accumulators, as the second.  Both maps of a
// differential head run side by side over one load of the values; the combination, the norm and the
// gate happen in registers before the store.  DT: tiles of 16 value dims at most; KC: chunks of 32 key
// dims at most.  Pages hold a multiple of 64 positions, dim is a multiple of 8, vdim of 16.
template <int MAPS, int DT, int KC>
__global__ void __launch_bounds__(64)
masked_attention_mfma_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache, const int32_t* __restrict__ block_table,
                             int table_stride, const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                             const float* __restrict__ gate, long gate_stride, bf16_t* __restrict__ out,
                             const int32_t* __restrict__ tiles, int heads, int kv_heads, int dim, int vdim, int page_size,
                             int mask_kind, int mask_size, float scale, float softcap, float lambda, float out_scale, float eps) {
  constexpr int QMAP = KC * 32, QROW = MAPS * QMAP + 8;      // rows 16 bytes longer than their chunks: 16 rows, 16 banks apart
  __shared__ __align__(16) bf16_t qs[16 * QROW];
  const int lane = threadIdx.x, j = lane & 15, g = lane >> 4;
  const int grp = heads / kv_heads;
  const int t0 = tiles ? tiles[2 * blockIdx.x] : (int)blockIdx.x, n = tiles ? tiles[2 * blockIdx.x + 1] : 1;
  int gk, h0, ncols;
  if (n == 1) {
    const int hc = grp < 16 ? grp : 16, per_kv = (grp + hc - 1) / hc;
    if ((int)blockIdx.y >= kv_heads * per_kv) return;
    gk = blockIdx.y / per_kv;
    const int first = (blockIdx.y % per_kv) * hc;
    h0 = gk * grp + first;
    ncols = min(hc, grp - first);
  } else {
    h0 = blockIdx.y;
    gk = h0 / grp;
    ncols = n;
  }
  const int qw = MAPS * dim;
  for (int idx = lane; idx < 16 * MAPS * KC * 4; idx += 64) {
    const int col = idx / (MAPS * KC * 4), rest = idx % (MAPS * KC * 4), mp = rest / (KC * 4), sl = rest % (KC * 4);
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (col < ncols && 8 * sl < dim) {
      const int tok = n == 1 ? t0 : t0 + col, head = n == 1 ? h0 + col : h0;
      v = *reinterpret_cast<const uint4*>(q + ((long)tok * heads + head) * qw + mp * dim + 8 * sl);
    }
    *reinterpret_cast<uint4*>(qs + col * QROW + mp * QMAP + 8 * sl) = v;
  }
  __syncthreads();
  const int my_tok = n == 1 ? t0 : t0 + j, my_head = n == 1 ? h0 + j : h0;
  const bool my_col = j < ncols;
  const int my_pos = my_col ? positions[my_tok] : -1;
  const int my_lo = my_col ? first_seen(my_pos, mask_kind, mask_size) : 0;
  const int pos_first = positions[t0], pos_last = pos_first + n - 1;
  const int lo_first = first_seen(pos_first, mask_kind, mask_size);
  const int32_t* pages = block_table + (long)seq_rows[t0] * table_stride;
  const int kw = kv_heads * MAPS * dim, kc = (dim + 31) / 32, dt_n = vdim / 16;
  const long page_elems = (long)page_size * (kw + kv_heads * vdim);
  const bf16_t* qlane = qs + j * QROW + 8 * g;
  ma_f32x4 acc[MAPS][DT];
  float m[MAPS], l[MAPS];
#pragma unroll
  for (int mp = 0; mp < MAPS; ++mp) {
    m[mp] = -INFINITY;
    l[mp] = 0.0f;
#pragma unroll
    for (int i = 0; i < DT; ++i) acc[mp][i] = ma_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  }
  for (int b = lo_first / 64; b <= pos_last / 64; ++b) {
    const int p0 = b * 64, in0 = p0 % page_size;
    const bf16_t* page = cache + (long)pages[p0 / page_size] * page_elems;
    const bf16_t* kbase = page + (long)in0 * kw + (long)gk * MAPS * dim + 8 * g;
    const bf16_t* vbase = page + (long)page_size * kw + (long)gk * vdim * page_size + in0 + 4 * g;
    uint4 pf[MAPS][2];
    float fold[MAPS];
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
      ma_f32x4 s[4];
#pragma unroll
      for (int pt = 0; pt < 4; ++pt) {
        s[pt] = ma_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        const bf16_t* krow = kbase + (long)(16 * pt + j) * kw + mp * dim;
        uint4 kf[KC];
#pragma unroll
        for (int c = 0; c < KC; ++c)
          kf[c] = (c < kc && 32 * c + 8 * g < dim) ? *reinterpret_cast<const uint4*>(krow + 32 * c) : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int c = 0; c < KC; ++c)
          if (c < kc)
            s[pt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                ma_frag(kf[c]), ma_frag(*reinterpret_cast<const uint4*>(qlane + mp * QMAP + 32 * c)), s[pt], 0, 0, 0);
      }
      float mx = -INFINITY;
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int p = p0 + 16 * pt + 4 * g + i;
          float v = s[pt][i] * scale;
          if (softcap > 0.0f) v = softcap * tanhf(v / softcap);
          v = (p >= my_lo && p <= my_pos) ? v : -INFINITY;
          s[pt][i] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m[mp], mx);
      const float m_safe = m_new == -INFINITY ? 0.0f : m_new;      // a column that has seen nothing yet
      fold[mp] = expf(m[mp] - m_safe);
      float sum = 0.0f;
#pragma unroll
      for (int pt = 0; pt < 4; ++pt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float w = expf(s[pt][i] - m_safe);        // 0 where the position is not seen
          s[pt][i] = w;
          sum += w;
        }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      l[mp] = fmaf(l[mp], fold[mp], sum);
      m[mp] = m_new;
#pragma unroll
      for (int c = 0; c < 2; ++c)
        pf[mp][c] = make_uint4(pack2_bf16(s[2 * c][0], s[2 * c][1]), pack2_bf16(s[2 * c][2], s[2 * c][3]),
                               pack2_bf16(s[2 * c + 1][0], s[2 * c + 1][1]), pack2_bf16(s[2 * c + 1][2], s[2 * c + 1][3]));
    }
    constexpr int VB = DT < 4 ? DT : 4;                         // tiles of 16 dims whose rows are asked for together
#pragma unroll
    for (int d0 = 0; d0 < DT; d0 += VB) {
      uint2 v[VB][4];
#pragma unroll
      for (int e = 0; e < VB; ++e) {
        if (d0 + e < dt_n) {
          const bf16_t* vrow = vbase + (long)(16 * (d0 + e) + j) * page_size;
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            v[e][2 * c] = *reinterpret_cast<const uint2*>(vrow + 32 * c);
            v[e][2 * c + 1] = *reinterpret_cast<const uint2*>(vrow + 32 * c + 16);
          }
        }
      }
#pragma unroll
      for (int e = 0; e < VB; ++e) {
        if (d0 + e < dt_n) {
#pragma unroll
          for (int mp = 0; mp < MAPS; ++mp) {
            acc[mp][d0 + e] *= fold[mp];
#pragma unroll
            for (int c = 0; c < 2; ++c)
              acc[mp][d0 + e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  ma_frag(make_uint4(v[e][2 * c].x, v[e][2 * c].y, v[e][2 * c + 1].x, v[e][2 * c + 1].y)), ma_frag(pf[mp][c]),
                  acc[mp][d0 + e], 0, 0, 0);
          }
        }
      }
    }
  }
  // a column's outputs: dims 16 dt + 4 g + i in the four lanes j, j + 16, j + 32, j + 48
  const float inv0 = 1.0f / l[0];
  float ss = 0.0f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    if (dt < dt_n) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float o = acc[0][dt][i] * inv0;
        if (MAPS == 2) {
          o = o - lambda * (acc[MAPS - 1][dt][i] * (1.0f / l[MAPS - 1]));
          ss = fmaf(o, o, ss);
        }
        acc[0][dt][i] = o;
      }
    }
  float norm = 1.0f;
  if (MAPS == 2) {
    ss += __shfl_xor(ss, 16, 64);
    ss += __shfl_xor(ss, 32, 64);
    norm = (1.0f / sqrtf(ss / (float)vdim + eps));
  }
  if (!my_col) return;
  bf16_t* dst = out + ((long)my_tok * heads + my_head) * vdim + 4 * g;
  const float* gsrc = gate ? gate + (long)my_tok * gate_stride + (long)my_head * vdim + 4 * g : nullptr;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    if (dt < dt_n) {
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        o[i] = acc[0][dt][i];
        if (MAPS == 2) o[i] = (o[i] * norm) * out_scale;
        if (gsrc) o[i] *= 1.0f / (1.0f + expf(-gsrc[16 * dt + i]));
      }
      *reinterpret_cast<uint2*>(dst + 16 * dt) = make_uint2(pack2_bf16(o[0], o[1]), pack2_bf16(o[2], o[3]));
    }
}

template <int MAPS, int DT, int KC>
static void launch_masked_mfma(const void* q, const void* cache, const int32_t* block_table, int table_stride,
                               const int32_t* positions, const int32_t* seq_rows, const float* gate, long gate_stride, void* out,
                               const int32_t* tiles, int n_tiles, int heads, int kv_heads, int dim, int vdim, int page_size,
                               int mask_kind, int mask_size, float scale, float softcap, float lambda, float out_scale, float eps,
                               hipStream_t stream) {
  masked_attention_mfma_kernel<MAPS, DT, KC><<<dim3(n_tiles, heads), 64, 0, stream>>>(
      (const bf16_t*)q, (const bf16_t*)cache, block_table, table_stride, positions, seq_rows, gate, gate_stride, (bf16_t*)out, tiles,
      heads, kv_heads, dim, vdim, page_size, mask_kind, mask_size, scale, softcap, lambda, out_scale, eps);
}
#endif

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
#if AXON_BF16
  return heads <= 65535 && dim % 8 == 0 && vdim % 16 == 0 && dim <= 256 && vdim <= 256 && page_size % 64 == 0;
#else
  return 0;
#endif
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
#if AXON_BF16
  if (axk_masked_attention_uses_mfma(heads, kv_heads, maps, dim, vdim, page_size) && ((uintptr_t)q & 15) == 0 &&
      ((uintptr_t)cache & 15) == 0 && ((uintptr_t)out & 7) == 0) {
    AXK_REQUIRE(tiles == nullptr || n_tiles > 0, "masked_attention: a list of %d tiles", n_tiles);
    const int nt = tiles ? n_tiles : n_tokens;
    const int size = dim > vdim ? dim : vdim;
#define MA_LAUNCH(MAPS, DT, KC)                                                                                                 \
  launch_masked_mfma<MAPS, DT, KC>(q, cache, block_table, table_stride, positions, seq_rows, gate, gate_stride, out, tiles, nt, \
                                   heads, kv_heads, dim, vdim, page_size, mask_kind, mask_size, scale, softcap, lambda,        \
                                   out_scale, eps, (hipStream_t)stream)
    if (maps == 1) {
      if (size <= 64) MA_LAUNCH(1, 4, 2); else if (size <= 128) MA_LAUNCH(1, 8, 4); else MA_LAUNCH(1, 16, 8);
    } else {
      if (size <= 64) MA_LAUNCH(2, 4, 2); else if (size <= 128) MA_LAUNCH(2, 8, 4); else MA_LAUNCH(2, 16, 8);
    }
#undef MA_LAUNCH
    AXK_LAUNCH_CHECK("masked_attention");
    return 0;
  }
#endif
  const long items = (long)n_tokens * heads;
  const size_t lds = (size_t)maps * dim * MA_WAVES * sizeof(float);
  masked_attention_kernel<<<(unsigned)((items + MA_WAVES - 1) / MA_WAVES), MA_WAVES * 64, lds, (hipStream_t)stream>>>(
      (const elem_t*)q, (const elem_t*)cache, block_table, table_stride, positions, seq_rows, gate, gate_stride, (elem_t*)out,
      n_tokens, heads, kv_heads, maps, dim, vdim, page_size, mask_kind, mask_size, scale, softcap, lambda, out_scale, eps);
  AXK_LAUNCH_CHECK("masked_attention");
  return 0;
}
