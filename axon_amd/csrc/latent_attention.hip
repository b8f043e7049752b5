// Attention over a latent cache: every position keeps one normed latent vector c (rank floats'
// worth, shared by all heads) and one rotated key part (rot floats' worth, shared too).  A head's
// unrotated key is Wuk c and its value Wuv c; neither is ever built.  The query's unrotated part
// is carried into the latent space instead (q_lat = Wuk^T q, a per-head product), so that
//     score(i, j) = (q_lat_i . c_j + q_rot_i . k_rot_j) scale,      o_lat_i = sum_j p_ij c_j,
// and the head's output is Wuv o_lat (another per-head product).  A page of the cache is
// [page_size][rank + rot] in the compute dtype.  Scores, weights and sums are 32-bit.
#include "api.h"
#include "common.h"

namespace {

// One block per token.  fused [T, stride] float32 holds the down projections' results:
//   [q_at, q_at + q_rank): the query latent -> RMS norm with q_gain -> cq [T, q_rank] (compute dtype);
//   [kv_at, kv_at + rank): the key/value latent -> RMS norm with kv_gain -> the page;
//   [kv_at + rank, + rot): the shared key part -> rotate-half on its first rot_dims dims -> the page.
// The sums of squares: a strided chain per thread, a butterfly per wave, the four waves in order.
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const float* __restrict__ fused, long stride, int q_at, int q_rank, int kv_at, int rank, int rot,
                      int rot_dims, const void* __restrict__ q_gain, int q_gain_is_f32, const void* __restrict__ kv_gain,
                      int kv_gain_is_f32, float eps, const float* __restrict__ table, const int32_t* __restrict__ positions,
                      const int32_t* __restrict__ seq_rows, const int32_t* __restrict__ block_table, int table_stride,
                      elem_t* __restrict__ cache, int page_size, elem_t* __restrict__ cq, int write_kv) {
  __shared__ float partial[4];
  const int t = blockIdx.x;
  const float* row = fused + (long)t * stride;
  if (q_rank > 0) {
    float ss = 0.0f;
    for (int i = threadIdx.x; i < q_rank; i += 256) ss = fmaf(row[q_at + i], row[q_at + i], ss);
    const float inv = 1.0f / sqrtf(block_sum_256(ss, partial) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += 256)
      cq[(long)t * q_rank + i] = from_float((row[q_at + i] * inv) * load_vec(q_gain, q_gain_is_f32, i));
    __syncthreads();
  }
  if (!write_kv) return;
  const int pos = positions[t];
  const int page = block_table[(long)seq_rows[t] * table_stride + pos / page_size];
  elem_t* dst = cache + ((long)page * page_size + pos % page_size) * (rank + rot);
  float ss = 0.0f;
  for (int i = threadIdx.x; i < rank; i += 256) ss = fmaf(row[kv_at + i], row[kv_at + i], ss);
  const float inv = 1.0f / sqrtf(block_sum_256(ss, partial) / (float)rank + eps);
  for (int i = threadIdx.x; i < rank; i += 256)
    dst[i] = from_float((row[kv_at + i] * inv) * load_vec(kv_gain, kv_gain_is_f32, i));
  const float* kr = row + kv_at + rank;
  const int half = rot_dims / 2;
  const float* tab = table + (long)t * half * 2;
  for (int i = threadIdx.x; i < half; i += 256) {
    const float s = tab[2 * i], c = tab[2 * i + 1];
    const float a = kr[i], b = kr[i + half];
    dst[rank + i] = from_float(__fsub_rn(__fmul_rn(a, c), __fmul_rn(b, s)));
    dst[rank + i + half] = from_float(__fadd_rn(__fmul_rn(b, c), __fmul_rn(a, s)));
  }
  for (int i = rot_dims + threadIdx.x; i < rot; i += 256) dst[rank + i] = from_float(kr[i]);
}

// The rotated part of every head's query: q [T, heads, dim + rot] float32 -> q_full [T, heads,
// rank + rot] float32, places rank .. rank + rot - 1 (the first `rank` are the per-head product's).
__global__ void latent_query_rope_kernel(const float* __restrict__ q, int dim, int rot, int rot_dims,
                                         const float* __restrict__ table, float* __restrict__ q_full, int rank, int heads) {
  const int t = blockIdx.x;
  const int half = rot_dims / 2;
  const float* tab = table + (long)t * half * 2;
  for (int idx = threadIdx.x; idx < heads * rot; idx += blockDim.x) {
    const int h = idx / rot, i = idx % rot;
    const float* src = q + ((long)t * heads + h) * (dim + rot) + dim;
    float v;
    if (i < half) v = __fsub_rn(__fmul_rn(src[i], tab[2 * i + 1]), __fmul_rn(src[i + half], tab[2 * i]));
    else if (i < rot_dims) v = __fadd_rn(__fmul_rn(src[i], tab[2 * (i - half) + 1]), __fmul_rn(src[i - half], tab[2 * (i - half)]));
    else v = src[i];
    q_full[((long)t * heads + h) * (rank + rot) + rank + i] = v;
  }
}

// One wave per (token, head), four waves a block.  Positions lo ..= pos in blocks of 64 aligned
// to absolute position, ascending; in a block lane j scores position 64 b + j (walking its key
// row against the query in LDS), the block's maximum and sum are butterflies, and the running
// (m, l, o) are rescaled block by block.  For the values lane d owns the latent dims d, d + 64, ...
// and walks the block's positions, taking each weight from its lane.
#define LA_WAVES 4
__global__ void __launch_bounds__(LA_WAVES * 64)
latent_attention_kernel(const float* __restrict__ q_full, const elem_t* __restrict__ cache,
                        const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ positions,
                        const int32_t* __restrict__ seq_rows, float* __restrict__ o_lat, int n_tokens, int heads, int rank,
                        int rot, int page_size, int window, float scale) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int width = rank + rot;
  const long item = (long)blockIdx.x * LA_WAVES + wave;
  const bool active = item < (long)n_tokens * heads;
  const int t = active ? (int)(item / heads) : 0, h = active ? (int)(item % heads) : 0;
  float* qs = smem + (long)wave * width;
  const float* qsrc = q_full + ((long)t * heads + h) * width;
  if (active)
    for (int i = lane; i < width; i += 64) qs[i] = qsrc[i];
  __syncthreads();
  if (!active) return;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int32_t* pages = block_table + (long)seq_rows[t] * table_stride;
  constexpr int MAX_OWN = 16;                      // latent dims a lane owns: rank up to 1024
  float acc[MAX_OWN];
#pragma unroll
  for (int i = 0; i < MAX_OWN; ++i) acc[i] = 0.0f;
  float m = -INFINITY, l = 0.0f;
  for (int b = lo / 64; b <= pos / 64; ++b) {
    const int p = b * 64 + lane;
    const bool seen = p >= lo && p <= pos;
    float s = -INFINITY;
    if (seen) {
      const elem_t* key = cache + ((long)pages[p / page_size] * page_size + p % page_size) * width;
      float dot = 0.0f;
      for (int i = 0; i < width; ++i) dot = fmaf(qs[i], to_float(key[i]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float w = seen ? expf(s - m_new) : 0.0f;
    const float fold = expf(m - m_new);            // 0 at the first block (m = -inf)
    l = fmaf(l, fold, wave_sum(w));
    m = m_new;
#pragma unroll
    for (int i = 0; i < MAX_OWN; ++i) acc[i] *= fold;
    const int j_lo = max(lo, b * 64) - b * 64, j_hi = min(pos, b * 64 + 63) - b * 64;
    for (int j = j_lo; j <= j_hi; ++j) {
      const float wj = __shfl(w, j, 64);
      const int pj = b * 64 + j;
      const elem_t* val = cache + ((long)pages[pj / page_size] * page_size + pj % page_size) * width;
#pragma unroll
      for (int i = 0; i < MAX_OWN; ++i) {
        const int d = lane + 64 * i;
        if (d < rank) acc[i] = fmaf(wj, to_float(val[d]), acc[i]);
      }
    }
  }
  const float inv = 1.0f / l;
  float* dst = o_lat + ((long)t * heads + h) * rank;
#pragma unroll
  for (int i = 0; i < MAX_OWN; ++i) {
    const int d = lane + 64 * i;
    if (d < rank) dst[d] = acc[i] * inv;
  }
}

}  // namespace

extern "C" int axk_latent_prepare(const float* fused, long stride, int q_at, int q_rank, int kv_at, int rank, int rot,
                                  int rot_dims, const void* q_gain, int q_gain_is_f32, const void* kv_gain,
                                  int kv_gain_is_f32, float eps, const float* table, const int32_t* positions,
                                  const int32_t* seq_rows, const int32_t* block_table, int table_stride, void* cache,
                                  int page_size, void* cq, int n_tokens, int write_kv, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && q_rank >= 0 && rank > 0 && rot >= 0 && page_size > 0, "latent_prepare: bad sizes T=%d q_rank=%d "
              "rank=%d rot=%d page=%d", n_tokens, q_rank, rank, rot, page_size);
  AXK_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "latent_prepare: %d rotated dims of %d", rot_dims, rot);
  AXK_REQUIRE(q_at >= 0 && kv_at >= 0 && q_at + q_rank <= stride && kv_at + rank + rot <= stride,
              "latent_prepare: the parts do not fit rows of %ld", stride);
  if (n_tokens == 0) return 0;
  latent_prepare_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(fused, stride, q_at, q_rank, kv_at, rank, rot, rot_dims,
      q_gain, q_gain_is_f32, kv_gain, kv_gain_is_f32, eps, table, positions, seq_rows, block_table, table_stride,
      (elem_t*)cache, page_size, (elem_t*)cq, write_kv);
  AXK_LAUNCH_CHECK("latent_prepare");
  return 0;
}

extern "C" int axk_latent_query_rope(const float* q, int dim, int rot, int rot_dims, const float* table, float* q_full, int rank,
                                     int heads, int n_tokens, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && dim >= 0 && rot >= 0 && rank > 0 && heads > 0 && rot_dims % 2 == 0 && rot_dims <= rot,
              "latent_query_rope: bad sizes T=%d dim=%d rot=%d (%d rotated) rank=%d heads=%d", n_tokens, dim, rot, rot_dims,
              rank, heads);
  if (n_tokens == 0 || rot == 0) return 0;
  latent_query_rope_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(q, dim, rot, rot_dims, table, q_full, rank, heads);
  AXK_LAUNCH_CHECK("latent_query_rope");
  return 0;
}

extern "C" int axk_latent_attention(const float* q_full, const void* cache, const int32_t* block_table, int table_stride,
                                    const int32_t* positions, const int32_t* seq_rows, float* o_lat, int n_tokens, int heads,
                                    int rank, int rot, int page_size, int window, float scale, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && heads > 0 && rank > 0 && rot >= 0 && page_size > 0 && window >= 0,
              "latent_attention: bad sizes T=%d heads=%d rank=%d rot=%d page=%d window=%d", n_tokens, heads, rank, rot,
              page_size, window);
  AXK_REQUIRE(rank <= 1024, "latent_attention: a latent of %d dims (at most 1024)", rank);
  AXK_REQUIRE((long)(rank + rot) * LA_WAVES * 4 <= 64 * 1024, "latent_attention: keys of %d dims do not fit LDS", rank + rot);
  if (n_tokens == 0) return 0;
  const long items = (long)n_tokens * heads;
  const size_t lds = (size_t)(rank + rot) * LA_WAVES * sizeof(float);
  latent_attention_kernel<<<(unsigned)((items + LA_WAVES - 1) / LA_WAVES), LA_WAVES * 64, lds, (hipStream_t)stream>>>(
      q_full, (const elem_t*)cache, block_table, table_stride, positions, seq_rows, o_lat, n_tokens, heads, rank, rot,
      page_size, window, scale);
  AXK_LAUNCH_CHECK("latent_attention");
  return 0;
}
