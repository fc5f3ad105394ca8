// Mixers with a state of fixed size per request: a short causal convolution per channel,
// the real-gated linear recurrent unit, and the scalar-decay state-space recurrence.
//
// A request's state lives in float32 in its slot of a state array and is carried from step
// to step: a kernel starts from it, or from zero when the request's first token of the step
// is at position 0, and leaves it behind for the next step.  The batch is the flattened
// one of every step: q_start [R+1] bounds a request's tokens, positions [T] rise by one along
// them, token_req [T] is -1 for padding tokens (a padded request has one of those), slots [R]
// names the state row.  All arithmetic is float32; what a token computes depends on its
// request's earlier tokens only, not on how they were cut into steps nor on the batch.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

inline hipStream_t S(kvc_stream s) { return reinterpret_cast<hipStream_t>(s); }

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x * sigmoid_f(x); }
// log(1 + e^x) with no threshold: max(x, 0) + log1p(e^-|x|)
__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ------------------------------------------------------------- causal convolution
// out[t, c] = act(bias[c] + sum_j w[c, K-1-j] * in(p - j)), p the token's position; in(q) is 0
// for q < 0, this step's x for positions of this step, and the request's state (the K-1
// inputs before the step's first token) otherwise.  A thread per (token, channel).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    TO* __restrict__ out, int64_t out_stride, const TI* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, const float* __restrict__ bias, float* state,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, int C, int K, int act,
    int shift_state) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int t = blockIdx.x;
  if (c >= C) return;
  TO* o = out + static_cast<int64_t>(t) * out_stride + c;
  const int r = token_req[t];
  if (r < 0) {
    *o = from_float<TO>(0.f);
    return;
  }
  const int p = positions[t];
  const int i = t - q_start[r];
  float* st = state + static_cast<int64_t>(slots[r]) * (K - 1) * C + c;
  float acc = bias != nullptr ? bias[c] : 0.f;
  const float* wc = w + static_cast<int64_t>(c) * K;
  for (int j = 0; j < K && j <= p; ++j) {
    const float xv = (i - j >= 0) ? to_float(x[static_cast<int64_t>(t - j) * x_stride + c])
                                  : st[static_cast<int64_t>(K - 1 + i - j) * C];
    acc = fmaf(wc[K - 1 - j], xv, acc);
  }
  if (act == 1) acc = silu_f(acc);
  *o = from_float<TO>(acc);
  if (shift_state) {
    // the token is its request's only one in this step and this thread the only one that
    // touches the request's state of this channel: the state moves on here, in place
    for (int j = 0; j + 1 < K - 1; ++j) st[static_cast<int64_t>(j) * C] = st[static_cast<int64_t>(j + 1) * C];
    if (K > 1) st[static_cast<int64_t>(K - 2) * C] = to_float(x[static_cast<int64_t>(t) * x_stride + c]);
  }
}

// The same for up to 8 taps, eight consecutive tokens a thread: the taps' weights are fetched
// once, and the window of the last K inputs slides along in registers, so that a token costs
// one load of x and one store.
constexpr int kConvTokens = 8, kConvMaxTaps = 8;
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void causal_conv_window_kernel(
    TO* __restrict__ out, int64_t out_stride, const TI* __restrict__ x, int64_t x_stride,
    const float* __restrict__ w, const float* __restrict__ bias, const float* __restrict__ state,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, int T, int C, int K,
    int act) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int t0 = blockIdx.x * kConvTokens;
  if (c >= C) return;
  float wr[kConvMaxTaps], h[kConvMaxTaps];  // wr[j] weighs the input j positions back
#pragma unroll
  for (int j = 0; j < kConvMaxTaps; ++j) {
    wr[j] = j < K ? w[static_cast<int64_t>(c) * K + K - 1 - j] : 0.f;
    h[j] = 0.f;
  }
  const float b0 = bias != nullptr ? bias[c] : 0.f;
  bool sliding = false;  // h holds the window of the token before
  for (int tt = 0; tt < kConvTokens && t0 + tt < T; ++tt) {
    const int t = t0 + tt;
    TO* o = out + static_cast<int64_t>(t) * out_stride + c;
    const int r = token_req[t];
    if (r < 0) {
      *o = from_float<TO>(0.f);
      sliding = false;
      continue;
    }
    const int p = positions[t];
    const int i = t - q_start[r];
    if (sliding && i > 0) {  // the token before is the same request's, one position back
#pragma unroll
      for (int j = kConvMaxTaps - 1; j > 0; --j) h[j] = h[j - 1];
      h[0] = to_float(x[static_cast<int64_t>(t) * x_stride + c]);
    } else {
      const float* st = state + static_cast<int64_t>(slots[r]) * (K - 1) * C + c;
#pragma unroll
      for (int j = 0; j < kConvMaxTaps; ++j) {
        float v = 0.f;
        if (j < K && j <= p)
          v = (i - j >= 0) ? to_float(x[static_cast<int64_t>(t - j) * x_stride + c])
                           : st[static_cast<int64_t>(K - 1 + i - j) * C];
        h[j] = v;
      }
      sliding = true;
    }
    float acc = b0;
#pragma unroll
    for (int j = 0; j < kConvMaxTaps; ++j) acc = fmaf(wr[j], h[j], acc);
    if (act == 1) acc = silu_f(acc);
    *o = from_float<TO>(acc);
  }
}

// The state after the step: the last K-1 inputs.  A thread per (request, channel) moves what
// stays of the old state forward and appends the step's inputs; entry j only reads entries
// behind it, so rising j works in place.
template <typename TI>
__global__ __launch_bounds__(256) void conv_state_kernel(
    float* __restrict__ state, const TI* __restrict__ x, int64_t x_stride,
    const int32_t* __restrict__ token_req, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ slots, int C, int K) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int r = blockIdx.x;
  if (c >= C) return;
  const int b = q_start[r], n = q_start[r + 1] - b;
  if (n <= 0 || token_req[b] < 0) return;
  float* st = state + static_cast<int64_t>(slots[r]) * (K - 1) * C + c;
  for (int j = 0; j < K - 1; ++j) {
    const int i = n - (K - 1) + j;
    const float v = i >= 0 ? to_float(x[static_cast<int64_t>(b + i) * x_stride + c])
                           : st[static_cast<int64_t>(j + n) * C];
    st[static_cast<int64_t>(j) * C] = v;
  }
}

// ----------------------------------------------- gates of the linear recurrent unit
// The channels are cut into nb blocks of bw; in block b, r = sigmoid(Wa[b] u_b + ba) and
// i = sigmoid(Wi[b] u_b + bi) with square matrices [out, in].  Then log a = -c r softplus(lam),
// a = exp(log a), and the driven input sqrt(1 - a^2) i u, with 1 - a^2 taken as
// -expm1(2 log a).  A block of 256 threads owns 16 tokens x 64 outputs of one channel block
// and walks the inputs 32 at a time through LDS; each thread sums two dot products for four
// tokens in the order k = 0, 1, ...
constexpr int GT = 16, GK = 32;

// GO outputs a block and TPT = GO / 16 tokens a thread: 64 and 4 for many tokens; 16 and 1 for
// steps of few tokens, whose blocks are then four times as many (the weights, read once, are
// all the work there, and a launch of a few dozen blocks leaves most of the chip idle).
template <int GO, int TPT>
__global__ __launch_bounds__(256) void rglru_gates_kernel(
    float* __restrict__ a_out, float* __restrict__ drive, const float* __restrict__ u,
    const float* __restrict__ wa, const float* __restrict__ wi, const float* __restrict__ ba,
    const float* __restrict__ bi, const float* __restrict__ lam, float c_decay, int T, int W,
    int bw, int out_tiles) {
  static_assert(GO * (GT / TPT) == 256, "a thread per (output, group of tokens)");
  __shared__ float wa_s[GO][GK + 1];
  __shared__ float wi_s[GO][GK + 1];
  __shared__ float u_s[GT][GK];
  const int tid = threadIdx.x;
  const int t0 = blockIdx.x * GT;
  const int blk = blockIdx.y / out_tiles;
  const int o0 = (blockIdx.y - blk * out_tiles) * GO;
  const int ol = tid % GO;
  const int tg = tid / GO;
  const float* wa_b = wa + static_cast<int64_t>(blk) * bw * bw;
  const float* wi_b = wi + static_cast<int64_t>(blk) * bw * bw;
  float acc_a[TPT], acc_i[TPT];
#pragma unroll
  for (int tt = 0; tt < TPT; ++tt) acc_a[tt] = acc_i[tt] = 0.f;
  // a stage of 32 inputs is fetched into registers while the stage before it is multiplied
  constexpr int NW = GO * GK / 256, NU = GT * GK / 256;
  float wa_r[NW], wi_r[NW], u_r[NU];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int idx = tid + i * 256;
      const int row = idx / GK, col = idx - row * GK;
      const bool ok = o0 + row < bw && k0 + col < bw;
      const int64_t off = static_cast<int64_t>(o0 + row) * bw + k0 + col;
      wa_r[i] = ok ? wa_b[off] : 0.f;
      wi_r[i] = ok ? wi_b[off] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int idx = tid + i * 256;
      const int row = idx / GK, col = idx - row * GK;
      const bool ok = t0 + row < T && k0 + col < bw;
      u_r[i] = ok ? u[static_cast<int64_t>(t0 + row) * W + blk * bw + k0 + col] : 0.f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < bw; k0 += GK) {
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int idx = tid + i * 256;
      wa_s[idx / GK][idx % GK] = wa_r[i];
      wi_s[idx / GK][idx % GK] = wi_r[i];
    }
#pragma unroll
    for (int i = 0; i < NU; ++i) {
      const int idx = tid + i * 256;
      u_s[idx / GK][idx % GK] = u_r[i];
    }
    __syncthreads();
    if (k0 + GK < bw) fetch(k0 + GK);
#pragma unroll 8
    for (int k = 0; k < GK; ++k) {
      const float va = wa_s[ol][k], vi = wi_s[ol][k];
#pragma unroll
      for (int tt = 0; tt < TPT; ++tt) {
        const float uv = u_s[tg * TPT + tt][k];
        acc_a[tt] = fmaf(va, uv, acc_a[tt]);
        acc_i[tt] = fmaf(vi, uv, acc_i[tt]);
      }
    }
    __syncthreads();
  }
  if (o0 + ol >= bw) return;
  const int c = blk * bw + o0 + ol;
  const float sp = softplus_f(lam[c]);
  const float b_a = ba[c], b_i = bi[c];
#pragma unroll
  for (int tt = 0; tt < TPT; ++tt) {
    const int t = t0 + tg * TPT + tt;
    if (t >= T) continue;
    const float r = sigmoid_f(acc_a[tt] + b_a);
    const float g = sigmoid_f(acc_i[tt] + b_i);
    const float log_a = -c_decay * r * sp;
    const int64_t at = static_cast<int64_t>(t) * W + c;
    a_out[at] = expf(log_a);
    drive[at] = sqrtf(-expm1f(2.f * log_a)) * g * u[at];
  }
}

// S_t = a_t S_(t-1) + drive_t along each request's tokens, a thread per (request, channel);
// out_t = S_t * gelu_tanh(y_t).
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void rglru_scan_kernel(
    TO* __restrict__ out, const float* __restrict__ a, const float* __restrict__ drive,
    const TY* __restrict__ y, int64_t y_stride, float* __restrict__ state,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, int W) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int r = blockIdx.x;
  if (c >= W) return;
  const int b = q_start[r], e = q_start[r + 1];
  if (e <= b) return;
  if (token_req[b] < 0) {
    for (int t = b; t < e; ++t) out[static_cast<int64_t>(t) * W + c] = from_float<TO>(0.f);
    return;
  }
  float* st = state + static_cast<int64_t>(slots[r]) * W + c;
  float s = positions[b] == 0 ? 0.f : *st;
#pragma unroll 4
  for (int t = b; t < e; ++t) {
    const int64_t at = static_cast<int64_t>(t) * W + c;
    s = fmaf(a[at], s, drive[at]);
    out[at] = from_float<TO>(s * gelu_tanh_f(to_float(y[static_cast<int64_t>(t) * y_stride + c])));
  }
  *st = s;
}

// The same scan for long portions, cut into segments of 64 tokens so that a request's tokens are
// worked on side by side: the first kernel scans every segment from zero and leaves its decay
// product and its end value (and the request's state before the step); the second starts every
// segment from what the segments before it add up to, in their order, and writes the results.
constexpr int kScanSegment = 64;

__global__ __launch_bounds__(256) void rglru_segment_sums_kernel(
    float* __restrict__ ws, const float* __restrict__ a, const float* __restrict__ drive,
    const float* __restrict__ state, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ token_req, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ slots, int W, int segs) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int r = blockIdx.x / segs, sg = blockIdx.x - r * segs;
  if (c >= W) return;
  const int b = q_start[r], e = q_start[r + 1];
  const int t0 = b + sg * kScanSegment;
  if (t0 >= e || token_req[b] < 0) return;
  const int t1 = (t0 + kScanSegment < e) ? t0 + kScanSegment : e;
  float* out = ws + (static_cast<int64_t>(r) * (segs + 1) + sg) * 2 * W + c;
  if (sg == 0)  // the state before the step, where the second kernel finds it
    ws[(static_cast<int64_t>(r) * (segs + 1) + segs) * 2 * W + c] =
        positions[b] == 0 ? 0.f : state[static_cast<int64_t>(slots[r]) * W + c];
  float prod = 1.f, end = 0.f;
#pragma unroll 8
  for (int t = t0; t < t1; ++t) {
    const int64_t at = static_cast<int64_t>(t) * W + c;
    const float av = a[at];
    prod *= av;
    end = fmaf(av, end, drive[at]);
  }
  out[0] = prod;
  out[W] = end;
}

template <typename TY, typename TO>
__global__ __launch_bounds__(256) void rglru_scan_segments_kernel(
    TO* __restrict__ out, const float* __restrict__ a, const float* __restrict__ drive,
    const TY* __restrict__ y, int64_t y_stride, float* __restrict__ state,
    const float* __restrict__ ws, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, int W, int segs) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int r = blockIdx.x / segs, sg = blockIdx.x - r * segs;
  if (c >= W) return;
  const int b = q_start[r], e = q_start[r + 1];
  const int t0 = b + sg * kScanSegment;
  if (t0 >= e) return;
  const int t1 = (t0 + kScanSegment < e) ? t0 + kScanSegment : e;
  if (token_req[b] < 0) {
    for (int t = t0; t < t1; ++t) out[static_cast<int64_t>(t) * W + c] = from_float<TO>(0.f);
    return;
  }
  const float* sums = ws + static_cast<int64_t>(r) * (segs + 1) * 2 * W + c;
  float s = sums[static_cast<int64_t>(segs) * 2 * W];
  for (int j = 0; j < sg; ++j) s = fmaf(sums[static_cast<int64_t>(j) * 2 * W], s, sums[static_cast<int64_t>(j) * 2 * W + W]);
#pragma unroll 8
  for (int t = t0; t < t1; ++t) {
    const int64_t at = static_cast<int64_t>(t) * W + c;
    s = fmaf(a[at], s, drive[at]);
    out[at] = from_float<TO>(s * gelu_tanh_f(to_float(y[static_cast<int64_t>(t) * y_stride + c])));
  }
  if (t1 == e) state[static_cast<int64_t>(slots[r]) * W + c] = s;
}

// ------------------------------------------------------ state-space recurrence
// Per head h (group g = h / (heads / groups)), state S [N, P]:
//   dt = softplus(dt_raw + dt_bias[h]);  S = exp(-exp(A_log[h]) dt) S + dt B x^T;
//   y = S^T C + D[h] x.
// A block owns one (request, head, tile of PT value channels) and walks the request's tokens
// in order.  Thread (pl, ns) keeps the state elements S[n, p0 + pl] for n = ns, ns + 4, ... in
// registers; B, C, x and the step sizes of 16 tokens at a time are staged through LDS; the
// four partial sums over n of a y are added in the order ns = 0..3.
constexpr int SC = 16;  // tokens a stage
constexpr int NS = 4;   // threads that share a column of the state

template <int NPT, typename TD>
__global__ __launch_bounds__(256) void ssm_scan_kernel(
    float* __restrict__ y, const float* __restrict__ xbc, int64_t xbc_stride,
    const TD* __restrict__ dt_raw, int64_t dt_stride, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ state,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, int nh, int P, int N,
    int G, int PT) {
  extern __shared__ float lds[];
  float* b_s = lds;                    // [SC][N]
  float* c_s = b_s + SC * N;           // [SC][N]
  float* x_s = c_s + SC * N;           // [SC][PT]
  float* y_s = x_s + SC * PT;          // [SC][NS][PT]
  float* dt_s = y_s + SC * NS * PT;    // [SC]
  float* dec_s = dt_s + SC;            // [SC]
  const int r = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * PT;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int pl = tid % PT, ns = tid / PT;
  const int p = p0 + pl;
  const bool p_ok = p < P;
  const int inner = nh * P;
  const int b = q_start[r], e = q_start[r + 1];
  if (e <= b) return;
  if (token_req[b] < 0) {
    for (int idx = tid; idx < (e - b) * PT; idx += nthreads) {
      const int tt = idx / PT, q = p0 + idx - tt * PT;
      if (q < P) y[static_cast<int64_t>(b + tt) * inner + h * P + q] = 0.f;
    }
    return;
  }
  const int g = h / (nh / G);
  float* st = state + (static_cast<int64_t>(slots[r]) * nh + h) * N * P;
  const bool fresh = positions[b] == 0;
  float s[NPT];
#pragma unroll
  for (int k = 0; k < NPT; ++k) {
    const int n = ns + NS * k;
    s[k] = (!fresh && p_ok && n < N) ? st[static_cast<int64_t>(n) * P + p] : 0.f;
  }
  const float neg_a = -expf(a_log[h]);
  const float bias = dt_bias[h];
  const float skip = d_skip[h];
  const int off_b = inner + g * N, off_c = inner + G * N + g * N;
  for (int c0 = b; c0 < e; c0 += SC) {
    const int nt = (e - c0 < SC) ? e - c0 : SC;
    for (int idx = tid; idx < nt * N; idx += nthreads) {
      const int tt = idx / N, n = idx - tt * N;
      const float* row = xbc + static_cast<int64_t>(c0 + tt) * xbc_stride;
      b_s[tt * N + n] = row[off_b + n];
      c_s[tt * N + n] = row[off_c + n];
    }
    for (int idx = tid; idx < nt * PT; idx += nthreads) {
      const int tt = idx / PT, q = idx - tt * PT;
      x_s[tt * PT + q] = (p0 + q < P) ? xbc[static_cast<int64_t>(c0 + tt) * xbc_stride + h * P + p0 + q] : 0.f;
    }
    for (int tt = tid; tt < nt; tt += nthreads) {
      const float dt = softplus_f(to_float(dt_raw[static_cast<int64_t>(c0 + tt) * dt_stride + h]) + bias);
      dt_s[tt] = dt;
      dec_s[tt] = expf(neg_a * dt);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float dec = dec_s[tt];
      const float xv = x_s[tt * PT + pl] * dt_s[tt];
      const float* bt = b_s + tt * N;
      const float* ct = c_s + tt * N;
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < NPT; ++k) {
        const int n = ns + NS * k;
        if (n < N) {
          s[k] = fmaf(dec, s[k], bt[n] * xv);
          acc = fmaf(s[k], ct[n], acc);
        }
      }
      y_s[(tt * NS + ns) * PT + pl] = acc;
    }
    __syncthreads();
    for (int idx = tid; idx < nt * PT; idx += nthreads) {
      const int tt = idx / PT, q = idx - tt * PT;
      if (p0 + q >= P) continue;
      float v = 0.f;
#pragma unroll
      for (int z = 0; z < NS; ++z) v += y_s[(tt * NS + z) * PT + q];
      y[static_cast<int64_t>(c0 + tt) * inner + h * P + p0 + q] = fmaf(skip, x_s[tt * PT + q], v);
    }
    __syncthreads();
  }
  if (!p_ok) return;
#pragma unroll
  for (int k = 0; k < NPT; ++k) {
    const int n = ns + NS * k;
    if (n < N) st[static_cast<int64_t>(n) * P + p] = s[k];
  }
}

// The same recurrence for heads of 16 value channels and more (blocks of 256 threads over PT = 64
// or 16 of them; the narrow tiles where the wide ones would leave compute units idle), made for
// long portions: thread (pl, ns) keeps S[n, p0 + pl] for the NPT consecutive rows n = ns * NPT ..
// in registers; B and C lie in LDS padded with zeros to 4 * NPT rows, so that the inner loop has
// no bounds and reads them 16 bytes at a time; and while a stage of 16 tokens is worked on, the
// next stage's B, C, x and step sizes are already on their way from memory into registers (a
// block has one wave a SIMD and nothing else to hide that latency behind).
template <int NPT, int PT, typename TD>
__global__ __launch_bounds__(256) void ssm_scan_wide_kernel(
    float* __restrict__ y, const float* __restrict__ xbc, int64_t xbc_stride,
    const TD* __restrict__ dt_raw, int64_t dt_stride, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ state,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, int nh, int P, int N,
    int G) {
  constexpr int NSL = 256 / PT;            // threads that share a column of the state
  constexpr int NP = NSL * NPT;            // padded rows of the state
  constexpr int NB = SC * NP / 256;        // values of B (and of C) a thread fetches per stage
  constexpr int NX = (SC * PT + 255) / 256;
  static_assert(NPT % 4 == 0 && (SC * NP) % 256 == 0, "whole 16-byte reads and whole fetch rounds");
  __shared__ __attribute__((aligned(16))) float b_s[SC * NP];
  __shared__ __attribute__((aligned(16))) float c_s[SC * NP];
  __shared__ float x_s[SC * PT];
  __shared__ float y_s[SC * NSL * PT];
  __shared__ float dt_s[SC];
  __shared__ float dec_s[SC];
  const int r = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * PT;
  const int tid = threadIdx.x;
  const int pl = tid % PT, ns = tid / PT;
  const int p = p0 + pl;
  const bool p_ok = p < P;
  const int inner = nh * P;
  const int b = q_start[r], e = q_start[r + 1];
  if (e <= b) return;
  if (token_req[b] < 0) {
    for (int idx = tid; idx < (e - b) * PT; idx += 256) {
      const int tt = idx / PT, q = p0 + idx - tt * PT;
      if (q < P) y[static_cast<int64_t>(b + tt) * inner + h * P + q] = 0.f;
    }
    return;
  }
  const int g = h / (nh / G);
  float* st = state + (static_cast<int64_t>(slots[r]) * nh + h) * N * P;
  const bool fresh = positions[b] == 0;
  float s[NPT];
#pragma unroll
  for (int k = 0; k < NPT; ++k) {
    const int n = ns * NPT + k;
    s[k] = (!fresh && p_ok && n < N) ? st[static_cast<int64_t>(n) * P + p] : 0.f;
  }
  const float neg_a = -expf(a_log[h]);
  const float bias = dt_bias[h];
  const float skip = d_skip[h];
  const int off_b = inner + g * N, off_c = inner + G * N + g * N;

  float rb[NB], rc[NB], rx[NX], rdt = 0.f;
  auto fetch = [&](int c0) {  // the stage that starts at token c0, into registers
    const int nt = (e - c0 < SC) ? e - c0 : SC;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int idx = tid + i * 256;
      const int tt = idx / NP, n = idx - tt * NP;
      const bool ok = tt < nt && n < N;
      const float* row = xbc + static_cast<int64_t>(c0 + (ok ? tt : 0)) * xbc_stride;
      rb[i] = ok ? row[off_b + n] : 0.f;
      rc[i] = ok ? row[off_c + n] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int idx = tid + i * 256;
      const int tt = idx / PT, q = idx - tt * PT;
      const bool ok = idx < SC * PT && tt < nt && p0 + q < P;
      rx[i] = ok ? xbc[static_cast<int64_t>(c0 + tt) * xbc_stride + h * P + p0 + q] : 0.f;
    }
    rdt = tid < nt ? to_float(dt_raw[static_cast<int64_t>(c0 + tid) * dt_stride + h]) : 0.f;
  };
  auto stash = [&]() {  // registers to LDS
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      b_s[tid + i * 256] = rb[i];
      c_s[tid + i * 256] = rc[i];
    }
#pragma unroll
    for (int i = 0; i < NX; ++i)
      if (tid + i * 256 < SC * PT) x_s[tid + i * 256] = rx[i];
    if (tid < SC) {
      const float dt = softplus_f(rdt + bias);
      dt_s[tid] = dt;
      dec_s[tid] = expf(neg_a * dt);
    }
  };
  fetch(b);
  stash();
  __syncthreads();
  for (int c0 = b; c0 < e; c0 += SC) {
    const int nt = (e - c0 < SC) ? e - c0 : SC;
    const bool more = c0 + SC < e;
    if (more) fetch(c0 + SC);
    for (int tt = 0; tt < nt; ++tt) {
      const float dec = dec_s[tt];
      const float xv = x_s[tt * PT + pl] * dt_s[tt];
      const float4* bt = reinterpret_cast<const float4*>(b_s + tt * NP + ns * NPT);
      const float4* ct = reinterpret_cast<const float4*>(c_s + tt * NP + ns * NPT);
      float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
      for (int k4 = 0; k4 < NPT / 4; ++k4) {
        const float4 bv = bt[k4], cv = ct[k4];
        s[4 * k4 + 0] = fmaf(dec, s[4 * k4 + 0], bv.x * xv);
        s[4 * k4 + 1] = fmaf(dec, s[4 * k4 + 1], bv.y * xv);
        s[4 * k4 + 2] = fmaf(dec, s[4 * k4 + 2], bv.z * xv);
        s[4 * k4 + 3] = fmaf(dec, s[4 * k4 + 3], bv.w * xv);
        acc0 = fmaf(s[4 * k4 + 0], cv.x, acc0);
        acc1 = fmaf(s[4 * k4 + 1], cv.y, acc1);
        acc0 = fmaf(s[4 * k4 + 2], cv.z, acc0);
        acc1 = fmaf(s[4 * k4 + 3], cv.w, acc1);
      }
      y_s[(tt * NSL + ns) * PT + pl] = acc0 + acc1;
    }
    __syncthreads();
    for (int idx = tid; idx < nt * PT; idx += 256) {
      const int tt = idx / PT, q = idx - tt * PT;
      if (p0 + q >= P) continue;
      float v = 0.f;
#pragma unroll
      for (int z = 0; z < NSL; ++z) v += y_s[(tt * NSL + z) * PT + q];
      y[static_cast<int64_t>(c0 + tt) * inner + h * P + p0 + q] = fmaf(skip, x_s[tt * PT + q], v);
    }
    __syncthreads();
    if (more) {
      stash();
      __syncthreads();
    }
  }
  if (!p_ok) return;
#pragma unroll
  for (int k = 0; k < NPT; ++k) {
    const int n = ns * NPT + k;
    if (n < N) st[static_cast<int64_t>(n) * P + p] = s[k];
  }
}

// out[t, c] = gain[c] * v / sqrt(mean over c's group of v^2 + eps), v = y[t, c] * silu(z[t, c]):
// the gate first, then the norm in `groups` equal parts.  One block per (token, part).
template <typename TZ, typename TO>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_kernel(
    TO* __restrict__ out, const float* __restrict__ y, const TZ* __restrict__ z, int64_t z_stride,
    const float* __restrict__ gain, float eps, int width, int groups) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, part = blockIdx.y;
  const int n = width / groups;
  const int c0 = part * n;
  const float* yr = y + static_cast<int64_t>(t) * width + c0;
  const TZ* zr = z + static_cast<int64_t>(t) * z_stride + c0;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = yr[i] * silu_f(to_float(zr[i]));
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(n) + eps);
  TO* o = out + static_cast<int64_t>(t) * width + c0;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float v = yr[i] * silu_f(to_float(zr[i]));
    o[i] = from_float<TO>(v * inv * gain[c0 + i]);
  }
}

}  // namespace

// dtype codes: 0 float32, 1 bfloat16.
#define KVC_DISPATCH_2(code_a, TA, code_b, TB, ...)                         \
  do {                                                                      \
    if ((code_a) == 0 && (code_b) == 0) { using TA = float; using TB = float; __VA_ARGS__; }              \
    else if ((code_a) == 0 && (code_b) == 1) { using TA = float; using TB = kvc::bf16_t; __VA_ARGS__; }   \
    else if ((code_a) == 1 && (code_b) == 0) { using TA = kvc::bf16_t; using TB = float; __VA_ARGS__; }   \
    else if ((code_a) == 1 && (code_b) == 1) { using TA = kvc::bf16_t; using TB = kvc::bf16_t; __VA_ARGS__; } \
    else return kvc_fail("unknown dtype code");                             \
  } while (0)

extern "C" int kvc_causal_conv(void* out, int64_t out_stride, int out_dtype, const void* x,
                               int64_t x_stride, int x_dtype, const float* weight, const float* bias,
                               float* state, const int32_t* positions, const int32_t* token_req,
                               const int32_t* q_start, const int32_t* slots, int T, int R, int C,
                               int K, int act, int update_state, int single_tokens,
                               kvc_stream stream) {
  if (T < 0 || R < 0 || C <= 0 || K <= 0 || out_stride < C || x_stride < C)
    return kvc_fail("kvc_causal_conv: bad sizes");
  if (act != 0 && act != 1) return kvc_fail("kvc_causal_conv: activation 0 (none) or 1 (silu)");
  if (T == 0 || R == 0) return 0;
  const dim3 grid(T, (C + 255) / 256);
  if (grid.y > 65535u) return kvc_fail("kvc_causal_conv: too many channels for one launch");
  // steps of single tokens (the caller says so): the state moves on in the same kernel
  const int fused = (update_state && single_tokens && T == R) ? 1 : 0;
  if (!fused && K <= kConvMaxTaps && T >= 4 * kConvTokens && T >= 4 * static_cast<int64_t>(R)) {
    // portions of prompts (several tokens a request): eight tokens a thread, the window in
    // registers; single tokens of many requests would refill the window at every token
    const dim3 tiles((T + kConvTokens - 1) / kConvTokens, (C + 255) / 256);
    KVC_DISPATCH_2(x_dtype, TI, out_dtype, TO,
                   hipLaunchKernelGGL((causal_conv_window_kernel<TI, TO>), tiles, dim3(256), 0, S(stream),
                                      static_cast<TO*>(out), out_stride, static_cast<const TI*>(x),
                                      x_stride, weight, bias, state, positions, token_req, q_start,
                                      slots, T, C, K, act));
  } else {
    KVC_DISPATCH_2(x_dtype, TI, out_dtype, TO,
                   hipLaunchKernelGGL((causal_conv_kernel<TI, TO>), grid, dim3(256), 0, S(stream),
                                      static_cast<TO*>(out), out_stride, static_cast<const TI*>(x),
                                      x_stride, weight, bias, state, positions, token_req, q_start,
                                      slots, C, K, act, fused));
  }
  int rc = kvc_check_launch("kvc_causal_conv");
  if (rc != 0 || !update_state || K == 1 || fused) return rc;
  KVC_DISPATCH_DTYPE(x_dtype, TI,
                     hipLaunchKernelGGL((conv_state_kernel<TI>), dim3(R, (C + 255) / 256), dim3(256),
                                        0, S(stream), state, static_cast<const TI*>(x), x_stride,
                                        token_req, q_start, slots, C, K));
  return kvc_check_launch("kvc_causal_conv (state)");
}

extern "C" int kvc_rglru_gates(float* a_out, float* drive, const float* u, const float* wa,
                               const float* wi, const float* ba, const float* bi, const float* lam,
                               float c_decay, int T, int W, int nb, kvc_stream stream) {
  if (T < 0 || W <= 0 || nb <= 0 || W % nb) return kvc_fail("kvc_rglru_gates: bad sizes");
  if (T == 0) return 0;
  const int bw = W / nb;
  const bool few = T <= 16 * GT;  // few tokens: smaller tiles of outputs, four times the blocks
  const int go = few ? 16 : 64;
  const int out_tiles = (bw + go - 1) / go;
  const dim3 grid((T + GT - 1) / GT, nb * out_tiles);  // tokens on x, which has no 16-bit limit
  if (grid.y > 65535u) return kvc_fail("kvc_rglru_gates: too many channel tiles");
  if (few)
    hipLaunchKernelGGL((rglru_gates_kernel<16, 1>), grid, dim3(256), 0, S(stream), a_out, drive, u, wa,
                       wi, ba, bi, lam, c_decay, T, W, bw, out_tiles);
  else
    hipLaunchKernelGGL((rglru_gates_kernel<64, 4>), grid, dim3(256), 0, S(stream), a_out, drive, u, wa,
                       wi, ba, bi, lam, c_decay, T, W, bw, out_tiles);
  return kvc_check_launch("kvc_rglru_gates");
}

extern "C" int kvc_rglru_scan_segment(void) { return kScanSegment; }

extern "C" int kvc_rglru_scan(void* out, int out_dtype, const float* a, const float* drive,
                              const void* y, int64_t y_stride, int y_dtype, float* state,
                              const int32_t* positions, const int32_t* token_req,
                              const int32_t* q_start, const int32_t* slots, int R, int W,
                              int max_query_len, float* workspace, int64_t workspace_floats,
                              kvc_stream stream) {
  if (R < 0 || W <= 0 || y_stride < W) return kvc_fail("kvc_rglru_scan: bad sizes");
  if (R == 0) return 0;
  const unsigned tiles = (W + 255) / 256;
  if (tiles > 65535u) return kvc_fail("kvc_rglru_scan: too many channels for one launch");
  const int segs = (max_query_len + kScanSegment - 1) / kScanSegment;
  if (segs > 1 && workspace != nullptr) {
    // long portions: segments side by side, two kernels
    if (workspace_floats < static_cast<int64_t>(R) * (segs + 1) * 2 * W)
      return kvc_fail("kvc_rglru_scan: the workspace is too small");
    const dim3 grid(static_cast<unsigned>(R) * segs, tiles);
    hipLaunchKernelGGL(rglru_segment_sums_kernel, grid, dim3(256), 0, S(stream), workspace, a, drive,
                       state, positions, token_req, q_start, slots, W, segs);
    KVC_DISPATCH_2(y_dtype, TY, out_dtype, TO,
                   hipLaunchKernelGGL((rglru_scan_segments_kernel<TY, TO>), grid, dim3(256), 0, S(stream),
                                      static_cast<TO*>(out), a, drive, static_cast<const TY*>(y),
                                      y_stride, state, workspace, token_req, q_start, slots, W, segs));
    return kvc_check_launch("kvc_rglru_scan (segments)");
  }
  const dim3 grid(R, tiles);
  KVC_DISPATCH_2(y_dtype, TY, out_dtype, TO,
                 hipLaunchKernelGGL((rglru_scan_kernel<TY, TO>), grid, dim3(256), 0, S(stream),
                                    static_cast<TO*>(out), a, drive, static_cast<const TY*>(y),
                                    y_stride, state, positions, token_req, q_start, slots, W));
  return kvc_check_launch("kvc_rglru_scan");
}

extern "C" int kvc_ssm_scan_max_state(void) { return NS * 64; }

extern "C" int kvc_ssm_scan(float* y, const float* xbc, int64_t xbc_stride, const void* dt_raw,
                            int64_t dt_stride, int dt_dtype, const float* dt_bias,
                            const float* a_log, const float* d_skip, float* state,
                            const int32_t* positions, const int32_t* token_req,
                            const int32_t* q_start, const int32_t* slots, int R, int nh, int P, int N,
                            int G, kvc_stream stream) {
  if (R < 0 || nh <= 0 || P <= 0 || N <= 0 || G <= 0 || nh % G)
    return kvc_fail("kvc_ssm_scan: bad sizes");
  if (N > NS * 64) return kvc_fail("kvc_ssm_scan: a state of more than 256 rows a head");
  if (xbc_stride < static_cast<int64_t>(nh) * P + 2 * static_cast<int64_t>(G) * N || dt_stride < nh)
    return kvc_fail("kvc_ssm_scan: rows too short");
  if (R == 0) return 0;
  const int PT = P < 64 ? P : 64;
  const dim3 grid(R, nh, (P + PT - 1) / PT);
  if (grid.y > 65535u || grid.z > 65535u) return kvc_fail("kvc_ssm_scan: grid too large");
  const dim3 block(PT * NS);
  const size_t lds = sizeof(float) * (2 * SC * N + SC * PT + SC * NS * PT + 2 * SC);
  const int per_thread = (N + NS - 1) / NS;
#define KVC_SSM_LAUNCH(NPT)                                                                        \
  KVC_DISPATCH_DTYPE(dt_dtype, TD,                                                                 \
                     hipLaunchKernelGGL((ssm_scan_kernel<NPT, TD>), grid, block, lds, S(stream), y, \
                                        xbc, xbc_stride, static_cast<const TD*>(dt_raw), dt_stride, \
                                        dt_bias, a_log, d_skip, state, positions, token_req,       \
                                        q_start, slots, nh, P, N, G, PT))
#define KVC_SSM_LAUNCH_WIDE(NPT, PTW)                                                              \
  KVC_DISPATCH_DTYPE(dt_dtype, TD,                                                                 \
                     hipLaunchKernelGGL((ssm_scan_wide_kernel<NPT, PTW, TD>),                      \
                                        dim3(R, nh, (P + PTW - 1) / PTW), dim3(256), 0, S(stream), \
                                        y, xbc, xbc_stride, static_cast<const TD*>(dt_raw),        \
                                        dt_stride, dt_bias, a_log, d_skip, state, positions,       \
                                        token_req, q_start, slots, nh, P, N, G))
  // tiles of 16 value channels (sixteen threads a column of the state) where tiles of 64 would
  // give fewer blocks than the chip has compute units
  const int64_t wide_blocks = static_cast<int64_t>(R) * nh * ((P + 63) / 64);
  if (P >= 16 && (P < 64 || wide_blocks < kvc_device_compute_units())) {
    const int rows = (N + 15) / 16;
    if (rows <= 4) {
      KVC_SSM_LAUNCH_WIDE(4, 16);
    } else if (rows <= 8) {
      KVC_SSM_LAUNCH_WIDE(8, 16);
    } else {
      KVC_SSM_LAUNCH_WIDE(16, 16);
    }
  } else if (PT == 64) {  // heads of 64 value channels and more
    if (per_thread <= 16) {
      KVC_SSM_LAUNCH_WIDE(16, 64);
    } else if (per_thread <= 32) {
      KVC_SSM_LAUNCH_WIDE(32, 64);
    } else {
      KVC_SSM_LAUNCH_WIDE(64, 64);
    }
  } else if (per_thread <= 16) {
    KVC_SSM_LAUNCH(16);
  } else if (per_thread <= 32) {
    KVC_SSM_LAUNCH(32);
  } else {
    KVC_SSM_LAUNCH(64);
  }
#undef KVC_SSM_LAUNCH
#undef KVC_SSM_LAUNCH_WIDE
  return kvc_check_launch("kvc_ssm_scan");
}

extern "C" int kvc_gated_group_rmsnorm(void* out, int out_dtype, const float* y, const void* z,
                                       int64_t z_stride, int z_dtype, const float* gain, float eps,
                                       int T, int width, int groups, kvc_stream stream) {
  if (T < 0 || width <= 0 || groups <= 0 || width % groups || z_stride < width)
    return kvc_fail("kvc_gated_group_rmsnorm: bad sizes");
  if (T == 0) return 0;
  if (groups > 65535) return kvc_fail("kvc_gated_group_rmsnorm: too many parts");
  KVC_DISPATCH_2(z_dtype, TZ, out_dtype, TO,
                 hipLaunchKernelGGL((gated_group_rmsnorm_kernel<TZ, TO>), dim3(T, groups), dim3(256),
                                    0, S(stream), static_cast<TO*>(out), y,
                                    static_cast<const TZ*>(z), z_stride, gain, eps, width, groups));
  return kvc_check_launch("kvc_gated_group_rmsnorm");
}
