// A gated linear recurrence with a short causal convolution in front of it (the recurrent block of
// Griffin-like models): per-request state in 32-bit floats, carried from step to step.
//
// A request's state row holds two copies of ([channels] of recurrent state, then [taps - 1][channels]
// of the convolution's last inputs, oldest first); a new request starts from zeros, which is also
// what the convolution reads before the first token.  The state behind position p lives in copy
// p & 1: a step whose first position is s reads copy (s - 1) & 1 and writes the copy of its last
// position.  A step of one token therefore never writes what it read, and running it again (a
// decoding step is run once before it is captured into a graph) gives the same state and the same
// output.  The tokens of a request are contiguous in a step and a request is in a step once, so
// two tokens belong to one request iff their state slots (seq_rows) are equal.
#include "api.h"
#include "common.h"

namespace {

// u[t, c] = bias[c] + sum_k w[c, k] in(t - (taps - 1 - k)): the last column of w is the current
// token's.  One thread per (token, channel); inputs before the step come from the state.
__global__ void causal_conv_kernel(const elem_t* __restrict__ x, long x_stride, const elem_t* __restrict__ w,
                                   const void* __restrict__ bias, int bias_is_f32, const float* __restrict__ state,
                                   long state_stride, const int32_t* __restrict__ positions,
                                   const int32_t* __restrict__ seq_rows, float* __restrict__ u, int channels, int taps) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int slot = seq_rows[t];
  // how many earlier tokens of this step belong to the same request (up to taps - 1 matter)
  int inside = 0;
  while (inside < taps - 1 && t - inside - 1 >= 0 && seq_rows[t - inside - 1] == slot) ++inside;
  // the copy behind the position before the request's first of this step (not needed where all taps lie inside the step)
  const int before = (positions[t] - inside + 1) & 1;
  const float* kept = state + (long)slot * state_stride + (long)before * taps * channels + channels;      // [taps - 1][channels]
  float acc = 0.0f;
  for (int k = 0; k < taps; ++k) {
    const int back = taps - 1 - k;            // the input `back` tokens before this one
    float v;
    if (back <= inside) v = to_float(x[(long)(t - back) * x_stride + c]);
    else v = kept[(long)(taps - 1 - (back - inside)) * channels + c];        // the (back - inside)-th last kept input
    acc = fmaf(to_float(w[(long)c * taps + k]), v, acc);
  }
  if (bias) acc += load_vec(bias, bias_is_f32, c);
  u[(long)t * channels + c] = acc;
}

__device__ inline float sigmoid32(float z) { return 1.0f / (1.0f + expf(-z)); }

__device__ inline float gelu_tanh32(float z) {
  const float inner = 0.7978845608028654f * (z + 0.044715f * ((z * z) * z));
  return (0.5f * z) * (1.0f + tanhf(inner));
}

// One thread per (request of the step, channel), walking the request's tokens in order:
//   r = sigmoid(gates[t, r part]), i = sigmoid(gates[t, i part]), log a = -decay r softplus(lam),
//   S = a S + sqrt(1 - a^2) (i u), out[t] = S gelu(y[t]).
// gates [T, blocks, 2 block_width]: a block's r logits, then its i logits.  spans [n][3] = (slot,
// first token, tokens), or null: every token is a request of its own (a decoding step) in slot
// seq_rows[t].  Afterwards the request's state row holds S and the last taps - 1 inputs of the
// convolution.
__global__ void gated_scan_kernel(const float* __restrict__ gates, const float* __restrict__ u,
                                  const elem_t* __restrict__ y, long y_stride, const elem_t* __restrict__ x, long x_stride,
                                  const void* __restrict__ lam, int lam_is_f32, float decay, float* __restrict__ state,
                                  long state_stride, const int32_t* __restrict__ spans, const int32_t* __restrict__ positions,
                                  const int32_t* __restrict__ seq_rows, elem_t* __restrict__ out, int channels, int block_width,
                                  int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  int slot, first, count;
  if (spans) {
    slot = spans[3 * blockIdx.y]; first = spans[3 * blockIdx.y + 1]; count = spans[3 * blockIdx.y + 2];
  } else {
    slot = seq_rows[blockIdx.y]; first = blockIdx.y; count = 1;
  }
  const float l = load_vec(lam, lam_is_f32, c);
  const float softplus = l > 20.0f ? l : log1pf(expf(l));
  const float rate = -decay * softplus;
  const int b = c / block_width, j = c % block_width;
  const long gate_at = (long)b * 2 * block_width + j;
  const int start = positions[first];
  const float* from = state + (long)slot * state_stride + (long)((start + 1) & 1) * taps * channels;
  float* row = state + (long)slot * state_stride + (long)((start + count - 1) & 1) * taps * channels;
  float S = from[c];
  for (int t = first; t < first + count; ++t) {
    const float* g = gates + (long)t * 2 * channels + gate_at;
    const float r = sigmoid32(g[0]), i = sigmoid32(g[block_width]);
    const float log_a = rate * r;
    const float a = expf(log_a);
    const float mult = sqrtf(-expm1f(2.0f * log_a));                 // sqrt(1 - a^2), exact also where a is near 1
    S = fmaf(a, S, (mult * i) * u[(long)t * channels + c]);
    out[(long)t * channels + c] = from_float(S * gelu_tanh32(to_float(y[(long)t * y_stride + c])));
  }
  row[c] = S;
  // the convolution's last taps - 1 inputs: of (what was kept, this step's inputs) the last taps - 1;
  // place i takes what lies `count` places later (where both copies are one: read before it is written, ascending)
  float* kept = row + channels;
  const float* kept_from = from + channels;
  for (int i = 0; i < taps - 1; ++i) {
    const int at = i + count;
    kept[(long)i * channels + c] = at < taps - 1 ? kept_from[(long)at * channels + c]
                                                 : to_float(x[(long)(first + at - (taps - 1)) * x_stride + c]);
  }
}

// The same recurrence for long stretches of tokens, in two launches.  First, for every (token,
// channel) at once, what does not depend on the state: a, b = (sqrt(1 - a^2) i) u and gelu(y), the
// very operations of the kernel above, kept in 32-bit.  Then a thread per (request, channel) walks
// S = a S + b with sixteen steps' operands asked for ahead of the chain that needs them.  The bits
// are those of the kernel above.
__global__ void gated_scan_terms_kernel(const float* __restrict__ gates, const float* __restrict__ u,
                                        const elem_t* __restrict__ y, long y_stride, const void* __restrict__ lam,
                                        int lam_is_f32, float decay, float* __restrict__ terms, int channels, int block_width) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const float l = load_vec(lam, lam_is_f32, c);
  const float softplus = l > 20.0f ? l : log1pf(expf(l));
  const float rate = -decay * softplus;
  const int b = c / block_width, j = c % block_width;
  const float* g = gates + (long)t * 2 * channels + (long)b * 2 * block_width + j;
  const float r = sigmoid32(g[0]), i = sigmoid32(g[block_width]);
  const float log_a = rate * r;
  const float mult = sqrtf(-expm1f(2.0f * log_a));
  float* dst = terms + (long)t * 3 * channels + c;
  dst[0] = expf(log_a);
  dst[channels] = (mult * i) * u[(long)t * channels + c];
  dst[2 * channels] = gelu_tanh32(to_float(y[(long)t * y_stride + c]));
}

#define SCAN_AHEAD 16
__global__ void gated_scan_walk_kernel(const float* __restrict__ terms, const elem_t* __restrict__ x, long x_stride,
                                       float* __restrict__ state, long state_stride, const int32_t* __restrict__ spans,
                                       const int32_t* __restrict__ positions, elem_t* __restrict__ out, int channels, int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int slot = spans[3 * blockIdx.y], first = spans[3 * blockIdx.y + 1], count = spans[3 * blockIdx.y + 2];
  const int start = positions[first];
  const float* from = state + (long)slot * state_stride + (long)((start + 1) & 1) * taps * channels;
  float* row = state + (long)slot * state_stride + (long)((start + count - 1) & 1) * taps * channels;
  float S = from[c];
  int t = first;
  for (; t + SCAN_AHEAD <= first + count; t += SCAN_AHEAD) {
    float a[SCAN_AHEAD], b[SCAN_AHEAD], gy[SCAN_AHEAD];
#pragma unroll
    for (int i = 0; i < SCAN_AHEAD; ++i) {
      const float* src = terms + (long)(t + i) * 3 * channels + c;
      a[i] = src[0]; b[i] = src[channels]; gy[i] = src[2 * channels];
    }
#pragma unroll
    for (int i = 0; i < SCAN_AHEAD; ++i) {
      S = fmaf(a[i], S, b[i]);
      out[(long)(t + i) * channels + c] = from_float(S * gy[i]);
    }
  }
  for (; t < first + count; ++t) {
    const float* src = terms + (long)t * 3 * channels + c;
    S = fmaf(src[0], S, src[channels]);
    out[(long)t * channels + c] = from_float(S * src[2 * channels]);
  }
  row[c] = S;
  float* kept = row + channels;
  const float* kept_from = from + channels;
  for (int i = 0; i < taps - 1; ++i) {
    const int at = i + count;
    kept[(long)i * channels + c] = at < taps - 1 ? kept_from[(long)at * channels + c]
                                                 : to_float(x[(long)(first + at - (taps - 1)) * x_stride + c]);
  }
}

}  // namespace

extern "C" int axk_causal_conv(const void* x, long x_stride, const void* w, const void* bias, int bias_is_f32,
                               const float* state, long state_stride, const int32_t* positions, const int32_t* seq_rows,
                               float* u, int n_tokens, int channels, int taps, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && channels > 0 && taps >= 1 && x_stride >= channels,
              "causal_conv: bad sizes T=%d channels=%d taps=%d row stride %ld", n_tokens, channels, taps, x_stride);
  AXK_REQUIRE(state_stride >= 2L * taps * channels, "causal_conv: a state row of %ld floats does not hold 2 x %d x %d",
              state_stride, taps, channels);
  AXK_REQUIRE(n_tokens <= 65535, "causal_conv: %d tokens in one step (at most 65535)", n_tokens);
  if (n_tokens == 0) return 0;
  dim3 grid(ceil_div(channels, 256), n_tokens);
  causal_conv_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const elem_t*)x, x_stride, (const elem_t*)w, bias, bias_is_f32,
                                                           state, state_stride, positions, seq_rows, u, channels, taps);
  AXK_LAUNCH_CHECK("causal_conv");
  return 0;
}

extern "C" int axk_gated_scan(const float* gates, const float* u, const void* y, long y_stride, const void* x, long x_stride,
                              const void* lam, int lam_is_f32, float decay, float* state, long state_stride,
                              const int32_t* spans, int n_spans, const int32_t* positions, const int32_t* seq_rows, void* out,
                              int channels, int block_width, int taps, float* terms, int n_tokens, void* stream) {
  AXK_REQUIRE(n_spans >= 0 && channels > 0 && block_width > 0 && channels % block_width == 0 && taps >= 1,
              "gated_scan: bad sizes spans=%d channels=%d block width=%d taps=%d", n_spans, channels, block_width, taps);
  AXK_REQUIRE(state_stride >= 2L * taps * channels, "gated_scan: a state row of %ld floats does not hold 2 x %d x %d",
              state_stride, taps, channels);
  AXK_REQUIRE((spans != nullptr || seq_rows != nullptr) && positions != nullptr, "gated_scan: neither spans nor slots, or no positions");
  AXK_REQUIRE(n_spans <= 65535, "gated_scan: %d requests in one step (at most 65535)", n_spans);
  if (n_spans == 0) return 0;
  dim3 grid(ceil_div(channels, 64), n_spans);
  if (terms != nullptr && spans != nullptr && n_tokens > 0) {
    AXK_REQUIRE(n_tokens <= 65535, "gated_scan: %d tokens in one step (at most 65535)", n_tokens);
    dim3 wide(ceil_div(channels, 256), n_tokens);
    gated_scan_terms_kernel<<<wide, 256, 0, (hipStream_t)stream>>>(gates, u, (const elem_t*)y, y_stride, lam, lam_is_f32, decay,
                                                                  terms, channels, block_width);
    gated_scan_walk_kernel<<<grid, 64, 0, (hipStream_t)stream>>>(terms, (const elem_t*)x, x_stride, state, state_stride, spans,
                                                                positions, (elem_t*)out, channels, taps);
    AXK_LAUNCH_CHECK("gated_scan");
    return 0;
  }
  gated_scan_kernel<<<grid, 64, 0, (hipStream_t)stream>>>(gates, u, (const elem_t*)y, y_stride, (const elem_t*)x, x_stride, lam,
                                                         lam_is_f32, decay, state, state_stride, spans, positions,
                                                         seq_rows, (elem_t*)out, channels, block_width, taps);
  AXK_LAUNCH_CHECK("gated_scan");
  return 0;
}
