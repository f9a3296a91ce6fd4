// A norm without statistics, fused with the residual sum before it, and the squashing of logits.
//
//   add_tanhnorm:  resid += sa (sum_p A[p] + bias_a) + sb (sum_p B[p] + bias_b)
//                  out    = tanh(alpha resid) gain + shift          (alpha one number, gain and shift per column)
//   softcap:       x <- cap tanh(x / cap)
//
// Up to two pending terms, each the partial sums of a product with its bias and a factor of its
// own: a layer whose mixer and feed-forward read the same rows hands both on at once. With `rows`
// only the listed rows are normed, into a dense output, and `resid` stays as it was. All arithmetic
// is float32; the only rounding is the store of a 16-bit output.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

struct Term {
  const void* data;
  int dt, count;
  size_t stride;
  const void* bias;
  int bias_dt;
  float scale;
};

__device__ inline float term_at(const Term& t, size_t at, int col) {
  float d = 0.f;
  for (int p = 0; p < t.count; ++p) d += load_as_float(t.data, t.dt, p * t.stride + at);
  if (t.bias) d += load_as_float(t.bias, t.bias_dt, col);
  return d * t.scale;
}

__global__ __launch_bounds__(256) void add_tanhnorm_kernel(float* __restrict__ resid, Term a, Term b,
                                                           const void* __restrict__ alpha, int alpha_dt,
                                                           const void* __restrict__ gain, int gain_dt,
                                                           const void* __restrict__ shift, int shift_dt,
                                                           void* __restrict__ out, int out_dt,
                                                           const int* __restrict__ rows, int hidden) {
  const int r_out = blockIdx.x, r_in = rows ? rows[r_out] : r_out;
  const size_t irow = static_cast<size_t>(r_in) * hidden, orow = static_cast<size_t>(r_out) * hidden;
  const float al = load_as_float(alpha, alpha_dt, 0);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = resid[irow + i];
    if (a.data) v += term_at(a, irow + i, i);
    if (b.data) v += term_at(b, irow + i, i);
    if (!rows && a.data) resid[irow + i] = v;
    float y = tanhf(al * v) * load_as_float(gain, gain_dt, i);
    if (shift) y += load_as_float(shift, shift_dt, i);
    store_from_float(out, out_dt, orow + i, y);
  }
}

// Four columns a thread, an element's partial sums asked for together: the terms are float32 partial sums or
// 16-bit rows, the parameters share one element type, no bias is pending, everything starts on 16 bytes.
template <typename TA, typename TB, typename TP, typename TO>
__global__ __launch_bounds__(256) void add_tanhnorm_vec_kernel(float* __restrict__ resid, const TA* __restrict__ a,
                                                               int a_count, size_t a_stride, float a_scale,
                                                               const TB* __restrict__ b, int b_count, size_t b_stride,
                                                               float b_scale, const TP* __restrict__ alpha,
                                                               const TP* __restrict__ gain, const TP* __restrict__ shift,
                                                               TO* __restrict__ out, const int* __restrict__ rows,
                                                               int hidden) {
  const int r_out = blockIdx.x, r_in = rows ? rows[r_out] : r_out;
  const size_t irow = static_cast<size_t>(r_in) * hidden, orow = static_cast<size_t>(r_out) * hidden;
  const float al = to_float(alpha[0]);
  for (int i = 4 * threadIdx.x; i < hidden; i += 4 * blockDim.x) {
    float4 v = *reinterpret_cast<const float4*>(resid + irow + i);
    if (a) {
      const float4 d = sum_partials4(a + irow + i, a_stride, a_count);
      v.x += d.x * a_scale, v.y += d.y * a_scale, v.z += d.z * a_scale, v.w += d.w * a_scale;
    }
    if (b) {
      const float4 d = sum_partials4(b + irow + i, b_stride, b_count);
      v.x += d.x * b_scale, v.y += d.y * b_scale, v.z += d.z * b_scale, v.w += d.w * b_scale;
    }
    if (!rows && a) *reinterpret_cast<float4*>(resid + irow + i) = v;
    const float4 g = Vec4<TP>::load(gain + i);
    float4 y = {tanhf(al * v.x) * g.x, tanhf(al * v.y) * g.y, tanhf(al * v.z) * g.z, tanhf(al * v.w) * g.w};
    if (shift) y = add4(y, Vec4<TP>::load(shift + i));
    Vec4<TO>::store(out + orow + i, y);
  }
}

__global__ void softcap_kernel(float* __restrict__ x, size_t total, float cap) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < total) x[i] = cap * tanhf(x[i] / cap);
}

bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

}  // namespace

extern "C" int pyre_add_tanhnorm(float* resid, const void* a, int a_dt, int a_count, long a_stride, const void* a_bias,
                                 int a_bias_dt, float a_scale, const void* b, int b_dt, int b_count, long b_stride,
                                 const void* b_bias, int b_bias_dt, float b_scale, const void* alpha, const void* gain,
                                 const void* shift, int param_dt, void* out, int out_dt, const int* rows, int n,
                                 int hidden, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(param_dt) && known_dtype(out_dt), "add_tanhnorm: unknown dtype");
  PYRE_REQUIRE(!a || (known_dtype(a_dt) && a_count >= 1), "add_tanhnorm: bad first term");
  PYRE_REQUIRE(!b || (a && known_dtype(b_dt) && b_count >= 1), "add_tanhnorm: a second term needs a first one");
  PYRE_REQUIRE((!a_bias || known_dtype(a_bias_dt)) && (!b_bias || known_dtype(b_bias_dt)), "add_tanhnorm: unknown bias dtype");
  PYRE_REQUIRE(n >= 0 && hidden > 0 && alpha && gain, "add_tanhnorm: bad sizes n=%d hidden=%d", n, hidden);
  if (n == 0) return 0;
  const bool vec = hidden % 4 == 0 && !a_bias && !b_bias && a_stride % 4 == 0 && b_stride % 4 == 0 && aligned16(resid) &&
                   aligned16(a) && aligned16(b) && aligned16(gain) && aligned16(shift) && aligned16(out);
  if (vec) {
    const int threads = hidden >= 1024 ? 256 : hidden >= 512 ? 128 : 64;
    PYRE_DISPATCH(a ? a_dt : kF32, TA, PYRE_DISPATCH(b ? b_dt : kF32, TB, PYRE_DISPATCH(param_dt, TP, PYRE_DISPATCH(out_dt, TO,
        hipLaunchKernelGGL((add_tanhnorm_vec_kernel<TA, TB, TP, TO>), dim3(n), dim3(threads), 0, stream, resid,
                           static_cast<const TA*>(a), a_count, static_cast<size_t>(a_stride), a_scale,
                           static_cast<const TB*>(b), b_count, static_cast<size_t>(b_stride), b_scale,
                           static_cast<const TP*>(alpha), static_cast<const TP*>(gain), static_cast<const TP*>(shift),
                           static_cast<TO*>(out), rows, hidden)))));
    return check_launch("add_tanhnorm");
  }
  const Term ta{a, a_dt, a ? a_count : 0, static_cast<size_t>(a_stride), a_bias, a_bias_dt, a_scale};
  const Term tb{b, b_dt, b ? b_count : 0, static_cast<size_t>(b_stride), b_bias, b_bias_dt, b_scale};
  hipLaunchKernelGGL(add_tanhnorm_kernel, dim3(n), dim3(256), 0, stream, resid, ta, tb, alpha, param_dt, gain, param_dt,
                     shift, param_dt, out, out_dt, rows, hidden);
  return check_launch("add_tanhnorm");
}

extern "C" int pyre_softcap(float* x, long total, float cap, hipStream_t stream) {
  PYRE_REQUIRE(cap > 0.f, "softcap: the cap must be positive");
  if (total <= 0) return 0;
  hipLaunchKernelGGL(softcap_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, x, static_cast<size_t>(total), cap);
  return check_launch("softcap");
}
