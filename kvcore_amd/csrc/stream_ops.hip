// Kernels on rows of the residual stream that are not an RMS norm: layer norm with the
// residual sum, the mean of several branches that are each divided by their root mean
// square, two float32 row sets side by side as one operand of a product, a vector added to
// every row.  All arithmetic is float32; storage is float32 or bfloat16.

#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

namespace {

inline hipStream_t S(kvc_stream s) { return reinterpret_cast<hipStream_t>(s); }

// One block per row.  residual += delta; mean; mean of the squared deviations; then
// (x - mean) / sqrt(var + eps) * weight + bias.  Three passes over a row that stays in cache.
template <typename T>
__global__ __launch_bounds__(256) void add_layernorm_kernel(T* __restrict__ out,
                                                            float* __restrict__ residual,
                                                            const T* __restrict__ delta,
                                                            const float* __restrict__ weight,
                                                            const float* __restrict__ bias,
                                                            float eps, int H) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * H;
  float* r = residual + base;
  float sum = 0.f;
  if (delta != nullptr) {
    const T* dl = delta + base;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float v = r[i] + to_float(dl[i]);
      r[i] = v;
      sum += v;
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) sum += r[i];
  }
  const float mean = block_sum(sum, scratch) / static_cast<float>(H);
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float dv = r[i] - mean;
    ss = fmaf(dv, dv, ss);
  }
  const float var = block_sum(ss, scratch) / static_cast<float>(H);
  const float inv = 1.f / sqrtf(var + eps);
  T* o = out + base;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float b = bias != nullptr ? bias[i] : 0.f;
    o[i] = from_float<T>(fmaf((r[i] - mean) * inv, weight[i], b));
  }
}

// The same for rows of up to 256 * NV values, which a thread keeps in registers: residual and
// delta are read once and everything else is arithmetic and two block sums.
template <typename T, int NV>
__global__ __launch_bounds__(256) void add_layernorm_regs_kernel(T* __restrict__ out,
                                                                 float* __restrict__ residual,
                                                                 const T* __restrict__ delta,
                                                                 const float* __restrict__ weight,
                                                                 const float* __restrict__ bias,
                                                                 float eps, int H) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * H;
  float* r = residual + base;
  float v[NV], w[NV], sh[NV];  // gain and shift come with the row: one trip to memory in all
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * 256;
    v[i] = w[i] = sh[i] = 0.f;
    if (c < H) {
      v[i] = r[c];
      w[i] = weight[c];
      if (bias != nullptr) sh[i] = bias[c];
      if (delta != nullptr) {
        v[i] += to_float(delta[base + c]);
        r[c] = v[i];
      }
      sum += v[i];
    }
  }
  const float mean = block_sum(sum, scratch) / static_cast<float>(H);
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < H) {
      v[i] -= mean;
      ss = fmaf(v[i], v[i], ss);
    }
  }
  const float inv = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(H) + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < H) out[base + c] = from_float<T>(fmaf(v[i] * inv, w[i], sh[i]));
  }
}

constexpr int kMaxBranches = 4;
struct Branches {
  const float* x[kMaxBranches];
  const float* gain[kMaxBranches];
};

// out[t] = (1 / n) * sum_b gain_b * x_b[t] / sqrt(mean(x_b[t]^2) + eps).  One block per row.
// REGS: the rows (up to 256 * 8 values) and the gains are fetched once, all at the start, and
// kept in registers; otherwise a row is read twice.
template <typename T, bool REGS>
__global__ __launch_bounds__(256) void rms_branches_mean_kernel(T* __restrict__ out, Branches br,
                                                                int n, float eps, int H) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * H;
  const float share = 1.f / static_cast<float>(n);
  if constexpr (REGS) {
    constexpr int NV = 8;
    float x[kMaxBranches][NV], gn[kMaxBranches][NV], ss[kMaxBranches];
#pragma unroll
    for (int b = 0; b < kMaxBranches; ++b) {
      ss[b] = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int c = threadIdx.x + i * 256;
        const bool ok = b < n && c < H;
        x[b][i] = ok ? br.x[b][base + c] : 0.f;
        gn[b][i] = ok ? br.gain[b][c] : 0.f;
        ss[b] = fmaf(x[b][i], x[b][i], ss[b]);
      }
    }
    float acc[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = 0.f;
#pragma unroll
    for (int b = 0; b < kMaxBranches; ++b) {
      if (b < n) {  // uniform
        const float inv = 1.f / sqrtf(block_sum(ss[b], scratch) / static_cast<float>(H) + eps);
#pragma unroll
        for (int i = 0; i < NV; ++i) acc[i] = fmaf(x[b][i] * inv, gn[b][i], acc[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * 256;
      if (c < H) out[base + c] = from_float<T>(acc[i] * share);
    }
  } else {
    float inv[kMaxBranches];
    for (int b = 0; b < n; ++b) {
      const float* x = br.x[b] + base;
      float ss = 0.f;
      for (int i = threadIdx.x; i < H; i += blockDim.x) ss = fmaf(x[i], x[i], ss);
      inv[b] = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(H) + eps);
    }
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      float acc = 0.f;
      for (int b = 0; b < n; ++b) acc = fmaf(br.x[b][base + i] * inv[b], br.gain[b][i], acc);
      out[base + i] = from_float<T>(acc * share);
    }
  }
}

// out[t] = [a[t] | b[t]] rounded to T.
template <typename T>
__global__ void concat2_kernel(T* __restrict__ out, const float* __restrict__ a,
                               const float* __restrict__ b, int H, int64_t n) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t t = idx / (2 * H);
  const int c = static_cast<int>(idx - t * 2 * H);
  out[idx] = from_float<T>(c < H ? a[t * H + c] : b[t * H + (c - H)]);
}

__global__ void add_row_kernel(float* __restrict__ x, const float* __restrict__ v, int H, int64_t n) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  x[idx] += v[idx % H];
}

}  // namespace

extern "C" int kvc_add_layernorm(void* out, float* residual, const void* delta, const float* weight,
                                 const float* bias, float eps, int T, int H, int dtype,
                                 kvc_stream stream) {
  if (T < 0 || H <= 0) return kvc_fail("kvc_add_layernorm: bad sizes");
  if (T == 0) return 0;
  if (H <= 256 * 8) {
    KVC_DISPATCH_DTYPE(dtype, Tp,
                       hipLaunchKernelGGL((add_layernorm_regs_kernel<Tp, 8>), dim3(T), dim3(256), 0, S(stream),
                                          static_cast<Tp*>(out), residual,
                                          static_cast<const Tp*>(delta), weight, bias, eps, H));
    return kvc_check_launch("kvc_add_layernorm");
  }
  if (H <= 256 * 32) {
    KVC_DISPATCH_DTYPE(dtype, Tp,
                       hipLaunchKernelGGL((add_layernorm_regs_kernel<Tp, 32>), dim3(T), dim3(256), 0, S(stream),
                                          static_cast<Tp*>(out), residual,
                                          static_cast<const Tp*>(delta), weight, bias, eps, H));
    return kvc_check_launch("kvc_add_layernorm");
  }
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(add_layernorm_kernel<Tp>, dim3(T), dim3(256), 0, S(stream),
                                        static_cast<Tp*>(out), residual,
                                        static_cast<const Tp*>(delta), weight, bias, eps, H));
  return kvc_check_launch("kvc_add_layernorm");
}

extern "C" int kvc_rms_branches_mean(void* out, const float* const* host_x,
                                     const float* const* host_gain, int n, float eps, int T, int H,
                                     int dtype, kvc_stream stream) {
  if (T < 0 || H <= 0 || n <= 0 || n > kMaxBranches)
    return kvc_fail("kvc_rms_branches_mean: bad sizes (one to four branches)");
  if (T == 0) return 0;
  Branches br{};
  for (int b = 0; b < n; ++b) {
    br.x[b] = host_x[b];
    br.gain[b] = host_gain[b];
  }
  if (H <= 256 * 8)
    KVC_DISPATCH_DTYPE(dtype, Tp,
                       hipLaunchKernelGGL((rms_branches_mean_kernel<Tp, true>), dim3(T), dim3(256), 0,
                                          S(stream), static_cast<Tp*>(out), br, n, eps, H));
  else
    KVC_DISPATCH_DTYPE(dtype, Tp,
                       hipLaunchKernelGGL((rms_branches_mean_kernel<Tp, false>), dim3(T), dim3(256), 0,
                                          S(stream), static_cast<Tp*>(out), br, n, eps, H));
  return kvc_check_launch("kvc_rms_branches_mean");
}

extern "C" int kvc_concat2(void* out, const float* a, const float* b, int T, int H, int dtype,
                           kvc_stream stream) {
  if (T < 0 || H <= 0) return kvc_fail("kvc_concat2: bad sizes");
  const int64_t n = static_cast<int64_t>(T) * 2 * H;
  if (n == 0) return 0;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(concat2_kernel<Tp>, dim3(blocks), dim3(256), 0, S(stream),
                                        static_cast<Tp*>(out), a, b, H, n));
  return kvc_check_launch("kvc_concat2");
}

extern "C" int kvc_add_row(float* x, const float* v, int T, int H, kvc_stream stream) {
  if (T < 0 || H <= 0) return kvc_fail("kvc_add_row: bad sizes");
  const int64_t n = static_cast<int64_t>(T) * H;
  if (n == 0) return 0;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  hipLaunchKernelGGL(add_row_kernel, dim3(blocks), dim3(256), 0, S(stream), x, v, H, n);
  return kvc_check_launch("kvc_add_row");
}
