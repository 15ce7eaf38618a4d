// A causal convolution over time on each channel, for segments of sequences with a history per request.
//
//   y[t, c] = act(bias[c] + sum_j taps[c, j] * in(t - K + 1 + j, c))  (+ x[t, c] when `residual`)
//
// in(t', c) is the step's own row t' while t' lies inside the token's sequence portion; before the portion's start it
// is the request's history: state (slots, K - 1, C) float32 holds the last K - 1 inputs in their order in time (row
// K - 2 is the newest), zeros at a request's start.  act: 0 none, 1 silu.  The input may be a column range of wider
// rows (ldx, the range starts at x).  Products and sums are float32, taps from j = 0 upward, whatever the cut.
//
//   channel_conv         one thread per (token, channel), or per (token, eight channels) where widths and addresses
//                        allow 16-byte accesses (the same sums in the same order); a sequence that brings a single
//                        token also moves its history on (nobody else reads it in this step)
//   channel_conv_state   one thread per (sequence, channel), for the sequences that bring more than one token: the new
//                        history from the old one and the step's rows, read whole before anything is written
#include "common.h"

constexpr int CC_MAX_TAPS = 16;

template <typename TX, typename TO>
__global__ void channel_conv_kernel(const TX* __restrict__ x, int ldx, const float* __restrict__ taps,
                                    const float* __restrict__ bias, float* __restrict__ state,
                                    const int* __restrict__ seq_of_token, const int* __restrict__ q_start,
                                    const int* __restrict__ slots, TO* __restrict__ out, int ldo, int T, int C, int K,
                                    int act, int residual) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)T * C) return;
  const int t = (int)(i / C), c = (int)(i % C);
  const int s = seq_of_token[t];
  const int start = q_start[s], len = q_start[s + 1] - start;
  float* hist = state + (size_t)slots[s] * (K - 1) * C + c;
  float in[CC_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CC_MAX_TAPS; ++j) {
    if (j < K) {
      const int tt = t - (K - 1) + j;
      in[j] = tt >= start ? to_f32(x[(size_t)tt * ldx + c]) : hist[(size_t)(K - 1 + tt - start) * C];
    }
  }
  float y = bias ? bias[c] : 0.f;
#pragma unroll
  for (int j = 0; j < CC_MAX_TAPS; ++j)
    if (j < K) y = fmaf(taps[(size_t)c * K + j], in[j], y);
  if (act == 1) y = y / (1.f + expf(-y));
  if (residual) y += in[K - 1];
  out[(size_t)t * ldo + c] = from_f32<TO>(y);
  if (len == 1) {
#pragma unroll
    for (int j = 1; j < CC_MAX_TAPS; ++j)
      if (j < K) hist[(size_t)(j - 1) * C] = in[j];
  }
}

// Eight channels a thread; K is the number of taps, known at compile time: the thread's 8 K taps lie side by side in
// memory and are read as 16-byte pieces into registers.
template <typename TX, typename TO, int K>
__global__ void channel_conv_vec_kernel(const TX* __restrict__ x, int ldx, const float* __restrict__ taps,
                                        const float* __restrict__ bias, float* __restrict__ state,
                                        const int* __restrict__ seq_of_token, const int* __restrict__ q_start,
                                        const int* __restrict__ slots, TO* __restrict__ out, int ldo, int T, int C,
                                        int act, int residual) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int C8 = C / 8;
  if (i >= (long)T * C8) return;
  const int t = (int)(i / C8), c = (int)(i % C8) * 8;
  const int s = seq_of_token[t];
  const int start = q_start[s], len = q_start[s + 1] - start;
  float* hist = state + (size_t)slots[s] * (K - 1) * C + c;
  float w[8 * K];
#pragma unroll
  for (int q = 0; q < 2 * K; ++q) {
    const float4 v = reinterpret_cast<const float4*>(taps + (size_t)c * K)[q];
    w[4 * q] = v.x; w[4 * q + 1] = v.y; w[4 * q + 2] = v.z; w[4 * q + 3] = v.w;
  }
  float y[8], in[K][8];
  if (bias) load8f(bias + c, y);
  else {
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = 0.f;
  }
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const int tt = t - (K - 1) + j;
    if (tt >= start) load8f(x + (size_t)tt * ldx + c, in[j]);
    else load8f(hist + (size_t)(K - 1 + tt - start) * C, in[j]);
  }
#pragma unroll
  for (int j = 0; j < K; ++j) {
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = fmaf(w[e * K + j], in[j][e], y[e]);
  }
  if (len == 1) {
#pragma unroll
    for (int j = 1; j < K; ++j) store8f(hist + (size_t)(j - 1) * C, in[j]);     // (every row was read above)
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if (act == 1) y[e] = y[e] / (1.f + expf(-y[e]));
    if (residual) y[e] += in[K - 1][e];
  }
  store8f(out + (size_t)t * ldo + c, y);
}

template <typename TX>
__global__ void channel_conv_state_kernel(const TX* __restrict__ x, int ldx, float* __restrict__ state,
                                          const int* __restrict__ q_start, const int* __restrict__ slots, int nseq, int C,
                                          int K) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)nseq * C) return;
  const int s = (int)(i / C), c = (int)(i % C);
  const int start = q_start[s], len = q_start[s + 1] - start;
  if (len <= 1) return;                        // none, or moved on by the kernel above
  float* hist = state + (size_t)slots[s] * (K - 1) * C + c;
  float keep[CC_MAX_TAPS];
  // old history and new rows in a row: m < K - 1 is the history's row m, beyond it the step's row m - (K - 1); the new
  // history are the last K - 1 of them
#pragma unroll
  for (int j = 0; j < CC_MAX_TAPS - 1; ++j) {
    if (j < K - 1) {
      const int m = len + j;
      keep[j] = m < K - 1 ? hist[(size_t)m * C] : to_f32(x[(size_t)(start + m - (K - 1)) * ldx + c]);
    }
  }
#pragma unroll
  for (int j = 0; j < CC_MAX_TAPS - 1; ++j)
    if (j < K - 1) hist[(size_t)j * C] = keep[j];
}

extern "C" int gs_channel_conv(const void* x, int x_dtype, int ldx, const float* taps, const float* bias, float* state,
                               const int* seq_of_token, const int* q_start, const int* slots, void* out, int out_dtype,
                               int ldo, int T, int nseq, int C, int K, int act, int residual, int all_single,
                               hipStream_t stream) {
  GS_REQUIRE(T >= 0 && nseq >= 0 && C > 0 && K >= 1 && K <= CC_MAX_TAPS, "channel_conv: bad sizes T=%d C=%d taps=%d (at most %d)", T, C, K, CC_MAX_TAPS);
  GS_REQUIRE(ldx >= C && ldo >= C, "channel_conv: rows of %d and %d hold no %d channels", ldx, ldo, C);
  GS_REQUIRE(act == 0 || act == 1, "channel_conv: activation %d", act);
  if (T == 0) return 0;
  const bool vec = C % 8 == 0 && ldx % 8 == 0 && ldo % 8 == 0 && K <= 5 &&
                   (((uintptr_t)x | (uintptr_t)out | (uintptr_t)state | (uintptr_t)taps | (uintptr_t)bias) & 15) == 0;
  const int blocks = gs_ceil_div((long)T * (vec ? C / 8 : C), 256);
#define GS_VEC(TX, TO, KK)                                                                                              \
  channel_conv_vec_kernel<TX, TO, KK><<<blocks, 256, 0, stream>>>((const TX*)x, ldx, taps, bias, state, seq_of_token,   \
                                                                 q_start, slots, (TO*)out, ldo, T, C, act, residual)
#define GS_RUN(TX, TO)                                                                                                    \
  do {                                                                                                                    \
    if (vec && K == 1) GS_VEC(TX, TO, 1);                                                                                 \
    else if (vec && K == 2) GS_VEC(TX, TO, 2);                                                                            \
    else if (vec && K == 3) GS_VEC(TX, TO, 3);                                                                            \
    else if (vec && K == 4) GS_VEC(TX, TO, 4);                                                                            \
    else if (vec) GS_VEC(TX, TO, 5);                                                                                      \
    else                                                                                                                  \
      channel_conv_kernel<TX, TO><<<blocks, 256, 0, stream>>>((const TX*)x, ldx, taps, bias, state, seq_of_token, q_start, \
                                                             slots, (TO*)out, ldo, T, C, K, act, residual);               \
  } while (0)
  if (x_dtype == GS_F32 && out_dtype == GS_F32)
    GS_RUN(float, float);
  else if (x_dtype == GS_BF16 && out_dtype == GS_BF16)
    GS_RUN(bf16, bf16);
  else if (x_dtype == GS_BF16 && out_dtype == GS_F32)
    GS_RUN(bf16, float);
  else
    GS_REQUIRE(false, "channel_conv: unknown dtypes %d %d", x_dtype, out_dtype);
#undef GS_RUN
#undef GS_VEC
  GS_LAUNCH_CHECK("channel_conv");
  if (!all_single && K > 1) {
    const int sb = gs_ceil_div((long)nseq * C, 256);
    if (x_dtype == GS_F32)
      channel_conv_state_kernel<float><<<sb, 256, 0, stream>>>((const float*)x, ldx, state, q_start, slots, nseq, C, K);
    else
      channel_conv_state_kernel<bf16><<<sb, 256, 0, stream>>>((const bf16*)x, ldx, state, q_start, slots, nseq, C, K);
    GS_LAUNCH_CHECK("channel_conv_state");
  }
  return 0;
}
