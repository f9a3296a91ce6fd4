// A mixture of small feed-forward layers whose router squashes its logits one by one.
//
//   route_topk   z = the router product's partial sums, s = sigmoid(z); per token the `top` experts of largest
//                s (the lower index among equals), each weighted s / (sum of the chosen s + 1e-20); written as a
//                dense row gates[n, experts] (0 for an expert that is not chosen), float32. The experts are compared
//                by z, which orders them as s does and still tells two apart where both their s round to one.
//   expert_act   the experts' way up is one product over [W_0; W_1; ...; W_shared]; its result becomes
//                act[n, e ff + j] = gates[n, e] f(up[n, e ff + j]) for the routed experts and f(up) for the columns
//                of the shared expert behind them, f(u) = max(u, 0)^2. One product over
//                [W'_0 | W'_1 | ... | W'_shared] then gives the weighted sum of the chosen experts' results and the
//                shared expert's in one go.
//
// All arithmetic is float32.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

constexpr int kMaxPerLane = 8;  // experts a lane keeps: up to 512 experts

__global__ __launch_bounds__(kWave) void route_topk_kernel(const void* __restrict__ z, int z_dt, int n_partials,
                                                           size_t partial_stride, const void* __restrict__ bias,
                                                           int bias_dt, float* __restrict__ gates, int experts, int top) {
  const int n = blockIdx.x, lane = threadIdx.x;
  float s[kMaxPerLane], w[kMaxPerLane];  // s: the logits still to choose from
#pragma unroll
  for (int u = 0; u < kMaxPerLane; ++u) {
    const int e = lane + kWave * u;
    s[u] = -INFINITY, w[u] = 0.f;
    if (e < experts) {
      float v = 0.f;
      for (int p = 0; p < n_partials; ++p) v += load_as_float(z, z_dt, p * partial_stride + static_cast<size_t>(n) * experts + e);
      if (bias) v += load_as_float(bias, bias_dt, e);
      s[u] = fmaxf(v, -3.0e38f);  // finite, so that it beats the mark of an expert that is taken or not there
    }
  }
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = experts;
#pragma unroll
    for (int u = 0; u < kMaxPerLane; ++u)
      if (s[u] > best) best = s[u], at = lane + kWave * u;  // ascending index within the lane: the first of equals stays
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, kWave);
      const int oa = __shfl_xor(at, o, kWave);
      if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
    }
    const float score = 1.f / (1.f + expf(-best));
    total += score;
#pragma unroll
    for (int u = 0; u < kMaxPerLane; ++u)
      if (at == lane + kWave * u) w[u] = score, s[u] = -INFINITY;
  }
  const float inv = 1.f / (total + 1e-20f);
#pragma unroll
  for (int u = 0; u < kMaxPerLane; ++u) {
    const int e = lane + kWave * u;
    if (e < experts) gates[static_cast<size_t>(n) * experts + e] = w[u] * inv;
  }
}

__global__ __launch_bounds__(256) void expert_act_kernel(const void* __restrict__ up, int up_dt, int n_partials,
                                                         size_t partial_stride, const float* __restrict__ gates,
                                                         void* __restrict__ out, int out_dt, size_t total, int experts,
                                                         int ff, int width) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t n = i / width;
  const int c = static_cast<int>(i % width), e = c / ff;
  const float g = e < experts ? gates[n * experts + e] : 1.f;
  float y = 0.f;
  if (g != 0.f) {
    float u = 0.f;
    for (int p = 0; p < n_partials; ++p) u += load_as_float(up, up_dt, p * partial_stride + i);
    u = fmaxf(u, 0.f);
    y = g * (u * u);
  }
  store_from_float(out, out_dt, i, y);
}

// Four columns a thread (the experts' sizes, the shared expert's and the partial sums' stride are multiples of four,
// so the four share an expert); columns of an expert that the token does not take are not read.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void expert_act_vec_kernel(const TI* __restrict__ up, int n_partials, size_t partial_stride,
                                                             const float* __restrict__ gates, TO* __restrict__ out,
                                                             size_t total4, int experts, int ff, int width) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const int per_row = width / 4;
  const size_t n = i / per_row;
  const int c = 4 * static_cast<int>(i % per_row), e = c / ff;
  const float g = e < experts ? gates[n * experts + e] : 1.f;
  float4 y = {0.f, 0.f, 0.f, 0.f};
  if (g != 0.f) {
    const float4 u = sum_partials4(up + n * width + c, partial_stride, n_partials);
    const float a = fmaxf(u.x, 0.f), b = fmaxf(u.y, 0.f), cc = fmaxf(u.z, 0.f), d = fmaxf(u.w, 0.f);
    y = float4{g * (a * a), g * (b * b), g * (cc * cc), g * (d * d)};
  }
  Vec4<TO>::store(out + n * width + c, y);
}

}  // namespace

extern "C" int pyre_route_topk(const void* z, int z_dt, int n_partials, long partial_stride, const void* bias, int bias_dt,
                               float* gates, int n, int experts, int top, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(z_dt) && n_partials >= 1 && (!bias || known_dtype(bias_dt)), "route_topk: bad dtypes");
  PYRE_REQUIRE(experts > 0 && experts <= kWave * kMaxPerLane && top > 0 && top <= experts,
               "route_topk: %d of %d experts is not a choice this kernel makes", top, experts);
  if (n <= 0) return 0;
  hipLaunchKernelGGL(route_topk_kernel, dim3(n), dim3(kWave), 0, stream, z, z_dt, n_partials,
                     static_cast<size_t>(partial_stride), bias, bias_dt, gates, experts, top);
  return check_launch("route_topk");
}

extern "C" int pyre_expert_act(const void* up, int up_dt, int n_partials, long partial_stride, const float* gates, void* out,
                               int out_dt, int n, int experts, int ff, int shared_ff, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(up_dt) && known_dtype(out_dt) && n_partials >= 1, "expert_act: bad dtypes");
  PYRE_REQUIRE(experts > 0 && ff > 0 && shared_ff >= 0 && gates, "expert_act: bad sizes");
  if (n <= 0) return 0;
  const int width = experts * ff + shared_ff;
  const size_t total = static_cast<size_t>(n) * width;
  if (ff % 4 == 0 && shared_ff % 4 == 0 && partial_stride % 4 == 0 && reinterpret_cast<uintptr_t>(up) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    PYRE_DISPATCH(up_dt, TI, PYRE_DISPATCH(out_dt, TO,
        hipLaunchKernelGGL((expert_act_vec_kernel<TI, TO>), dim3((total / 4 + 255) / 256), dim3(256), 0, stream,
                           static_cast<const TI*>(up), n_partials, static_cast<size_t>(partial_stride), gates,
                           static_cast<TO*>(out), total / 4, experts, ff, width)));
    return check_launch("expert_act");
  }
  hipLaunchKernelGGL(expert_act_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, up, up_dt, n_partials,
                     static_cast<size_t>(partial_stride), gates, out, out_dt, total, experts, ff, width);
  return check_launch("expert_act");
}
