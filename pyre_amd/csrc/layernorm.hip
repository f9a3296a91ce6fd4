// Layer norm around the float32 residual stream, for blocks that norm a sublayer's result
// before it is added ("sandwich" blocks), a gated feed-forward activation with clipped inputs,
// and a scaling of float32 rows. All arithmetic float32.
//
//   d      = sum of the pending partial sums (+ bias)
//   y      = post ? LN(d; post_eps) * post_gain * post_scale : d       (the sublayer's own norm and layer scale)
//   resid += y
//   out    = LN(resid; eps) * gain
//   LN(x; e) = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + e)
//
// One block per row; a thread keeps its elements in registers (every 256th), so the row is read
// once. Mean and variance are two separate sums, the variance over the deviations from the mean.
// With `rows` only the listed rows are normed, into out[0 .. n), and resid is left as it was.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

constexpr int kThreads = 256;

template <int ITEMS>
__global__ __launch_bounds__(kThreads) void add_layernorm_kernel(
    float* __restrict__ resid, const void* __restrict__ delta, int delta_dt, int n_partials, size_t partial_stride,
    const void* __restrict__ bias, int bias_dt, const void* __restrict__ post_gain, int post_gain_dt,
    const void* __restrict__ post_scale, int post_scale_dt, float post_eps, const void* __restrict__ gain,
    int gain_dt, void* __restrict__ out, int out_dt, const int* __restrict__ rows, int hidden, float eps) {
  __shared__ float scratch[16];
  const int r_out = blockIdx.x, r_in = rows ? rows[r_out] : r_out, tid = threadIdx.x;
  const size_t row = static_cast<size_t>(r_in) * hidden;
  const float inv_n = 1.f / static_cast<float>(hidden);
  float v[ITEMS];

  // mean and 1 / sqrt(variance + e) of the row held in v
  auto stats = [&](float e, float& mean, float& inv) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      if (tid + k * kThreads < hidden) s += v[k];
    mean = block_sum(s, scratch) * inv_n;
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      if (tid + k * kThreads < hidden) ss += (v[k] - mean) * (v[k] - mean);
    inv = 1.f / sqrtf(block_sum(ss, scratch) * inv_n + e);
  };

  if (delta) {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = tid + k * kThreads;
      float d = 0.f;
      if (i < hidden) {
        for (int p = 0; p < n_partials; ++p) d += load_as_float(delta, delta_dt, p * partial_stride + row + i);
        if (bias) d += load_as_float(bias, bias_dt, i);
      }
      v[k] = d;
    }
    if (post_gain) {
      float mean, inv;
      stats(post_eps, mean, inv);
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) {
        const int i = tid + k * kThreads;
        if (i < hidden) {
          float y = (v[k] - mean) * inv * load_as_float(post_gain, post_gain_dt, i);
          if (post_scale) y *= load_as_float(post_scale, post_scale_dt, i);
          v[k] = y;
        }
      }
    }
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = tid + k * kThreads;
      if (i < hidden) {
        v[k] += resid[row + i];
        if (!rows) resid[row + i] = v[k];
      }
    }
  } else {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = tid + k * kThreads;
      v[k] = i < hidden ? resid[row + i] : 0.f;
    }
  }
  float mean, inv;
  stats(eps, mean, inv);
  const size_t orow = static_cast<size_t>(r_out) * hidden;
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const int i = tid + k * kThreads;
    if (i < hidden) store_from_float(out, out_dt, orow + i, (v[k] - mean) * inv * load_as_float(gain, gain_dt, i));
  }
}

// The same with four elements to a load (the row's width and the partial sums' stride are multiples
// of four, no bias), the partial sums of an element asked for together: a step of few rows is all
// waiting for loads. THREADS x ITEMS float4 hold a row.
template <typename TD, typename TG, typename TO, int THREADS, int ITEMS>
__global__ __launch_bounds__(THREADS) void add_layernorm_vec_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, int n_partials, size_t partial_stride,
    const TG* __restrict__ post_gain, const TG* __restrict__ post_scale, float post_eps, const TG* __restrict__ gain,
    TO* __restrict__ out, const int* __restrict__ rows, int hidden, float eps) {
  __shared__ float scratch[16];
  const int r_out = blockIdx.x, r_in = rows ? rows[r_out] : r_out, tid = threadIdx.x, quads = hidden / 4;
  const size_t row = static_cast<size_t>(r_in) * hidden;
  const float inv_n = 1.f / static_cast<float>(hidden);
  float4 v[ITEMS];
  auto stats = [&](float e, float& mean, float& inv) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      if (tid + k * THREADS < quads) s += (v[k].x + v[k].y) + (v[k].z + v[k].w);
    mean = block_sum(s, scratch) * inv_n;
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      if (tid + k * THREADS < quads) {
        const float a = v[k].x - mean, b = v[k].y - mean, c = v[k].z - mean, d = v[k].w - mean;
        ss += (a * a + b * b) + (c * c + d * d);
      }
    inv = 1.f / sqrtf(block_sum(ss, scratch) * inv_n + e);
  };
  if (delta) {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = 4 * (tid + k * THREADS);
      v[k] = i < hidden ? sum_partials4(delta + row + i, partial_stride, n_partials) : float4{0.f, 0.f, 0.f, 0.f};
    }
    if (post_gain) {
      float mean, inv;
      stats(post_eps, mean, inv);
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) {
        const int i = 4 * (tid + k * THREADS);
        if (i < hidden) {
          const float4 pg = Vec4<TG>::load(post_gain + i);
          float4 y = {(v[k].x - mean) * inv * pg.x, (v[k].y - mean) * inv * pg.y, (v[k].z - mean) * inv * pg.z,
                      (v[k].w - mean) * inv * pg.w};
          if (post_scale) {
            const float4 ps = Vec4<TG>::load(post_scale + i);
            y = float4{y.x * ps.x, y.y * ps.y, y.z * ps.z, y.w * ps.w};
          }
          v[k] = y;
        }
      }
    }
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = 4 * (tid + k * THREADS);
      if (i < hidden) {
        v[k] = add4(v[k], Vec4<float>::load(resid + row + i));
        if (!rows) Vec4<float>::store(resid + row + i, v[k]);
      }
    }
  } else {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const int i = 4 * (tid + k * THREADS);
      v[k] = i < hidden ? Vec4<float>::load(resid + row + i) : float4{0.f, 0.f, 0.f, 0.f};
    }
  }
  float mean, inv;
  stats(eps, mean, inv);
  const size_t orow = static_cast<size_t>(r_out) * hidden;
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const int i = 4 * (tid + k * THREADS);
    if (i < hidden) {
      const float4 gn = Vec4<TG>::load(gain + i);
      Vec4<TO>::store(out + orow + i, float4{(v[k].x - mean) * inv * gn.x, (v[k].y - mean) * inv * gn.y,
                                             (v[k].z - mean) * inv * gn.z, (v[k].w - mean) * inv * gn.w});
    }
  }
}

// act[n, i] = g * sigmoid(slope * (g + cubic g^3)) * (u + shift), g = min(gate[n, i], limit), u = clamp(up[n, i], -limit, limit);
// gate = gu[:, :I], up = gu[:, I:], the partial sums added first. limit <= 0: no clipping.
__global__ void clipped_glu_kernel(const void* __restrict__ gu, int gu_dt, int n_partials, size_t partial_stride,
                                   void* __restrict__ out, int out_dt, size_t total, int inter, float limit,
                                   float slope, float shift, float cubic) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t n = i / inter, c = i % inter;
  const size_t gi = n * 2 * inter + c, ui = gi + inter;
  float g = 0.f, u = 0.f;
  for (int p = 0; p < n_partials; ++p) {
    g += load_as_float(gu, gu_dt, p * partial_stride + gi);
    u += load_as_float(gu, gu_dt, p * partial_stride + ui);
  }
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  store_from_float(out, out_dt, i, g / (1.f + expf(-slope * fmaf(cubic * g, g * g, g))) * (u + shift));
}

__device__ inline float clipped_unit(float g, float u, float limit, float slope, float shift, float cubic) {
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return g / (1.f + expf(-slope * fmaf(cubic * g, g * g, g))) * (u + shift);
}

// The same, four elements a thread (inter and the partial sums' stride are multiples of four).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void clipped_glu_vec_kernel(const TI* __restrict__ gu, int n_partials, size_t partial_stride,
                                                              TO* __restrict__ out, size_t total4, int inter, float limit,
                                                              float slope, float shift, float cubic) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const int per_row = inter / 4;
  const size_t n = i / per_row, c = 4 * (i % per_row);
  const size_t gi = n * 2 * inter + c;
  const float4 g = sum_partials4(gu + gi, partial_stride, n_partials), u = sum_partials4(gu + gi + inter, partial_stride, n_partials);
  Vec4<TO>::store(out + n * inter + c, float4{clipped_unit(g.x, u.x, limit, slope, shift, cubic), clipped_unit(g.y, u.y, limit, slope, shift, cubic),
                                              clipped_unit(g.z, u.z, limit, slope, shift, cubic), clipped_unit(g.w, u.w, limit, slope, shift, cubic)});
}

// The same for many rows of bfloat16 in and out without partial sums to add: eight elements a thread,
// loads that pass the caches (the rows are read once), the hardware's exponential and reciprocal (the
// result is rounded to bfloat16 anyway).
__global__ __launch_bounds__(256) void clipped_glu_stream_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out,
                                                                 size_t total8, int inter, float limit, float slope,
                                                                 float shift, float cubic) {
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int per_row = inter / 8;
  const size_t n = i / per_row, c = 8 * (i % per_row);
  const bf16* gp = gu + n * 2 * inter + c;
  const u32x4 g = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(gp));
  const u32x4 u = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(gp + inter));
  auto unit = [&](float gv, float uv) {
    if (limit > 0.f) {
      gv = fminf(gv, limit);
      uv = fminf(fmaxf(uv, -limit), limit);
    }
    return gv * __builtin_amdgcn_rcpf(1.f + __expf(-slope * fmaf(cubic * gv, gv * gv, gv))) * (uv + shift);
  };
  u32x4 y;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    y[j] = pack_bf16x2(unit(__uint_as_float(g[j] << 16), __uint_as_float(u[j] << 16)),
                       unit(__uint_as_float(g[j] & 0xffff0000u), __uint_as_float(u[j] & 0xffff0000u)));
  *reinterpret_cast<u32x4*>(out + n * inter + c) = y;
}

__global__ void scale_kernel(float* __restrict__ x, size_t total, float s) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < total) x[i] *= s;
}

}  // namespace

extern "C" int pyre_add_layernorm(float* resid, const void* delta, int delta_dt, int n_partials, long partial_stride,
                                  const void* bias, int bias_dt, const void* post_gain, int post_gain_dt,
                                  const void* post_scale, int post_scale_dt, float post_eps, const void* gain,
                                  int gain_dt, void* out, int out_dt, const int* rows, int n, int hidden, float eps,
                                  hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(gain_dt) && known_dtype(out_dt), "add_layernorm: unknown dtype");
  PYRE_REQUIRE(!delta || (known_dtype(delta_dt) && n_partials >= 1), "add_layernorm: bad delta (dtype %d, partials %d)",
               delta_dt, n_partials);
  PYRE_REQUIRE(!bias || known_dtype(bias_dt), "add_layernorm: unknown bias dtype");
  PYRE_REQUIRE(!post_gain || (delta && known_dtype(post_gain_dt) && post_eps > 0.f),
               "add_layernorm: a norm of the pending term needs the term, a gain and a positive eps");
  PYRE_REQUIRE(!post_scale || (post_gain && known_dtype(post_scale_dt)), "add_layernorm: a layer scale without its norm");
  PYRE_REQUIRE(n >= 0 && hidden > 0 && eps > 0.f, "add_layernorm: bad sizes n=%d hidden=%d", n, hidden);
  PYRE_REQUIRE(hidden <= 64 * kThreads, "add_layernorm: rows of %d elements are more than %d", hidden, 64 * kThreads);
  if (n == 0) return 0;
  const bool same_gains = (!post_gain || post_gain_dt == gain_dt) && (!post_scale || post_scale_dt == gain_dt);
  if (!bias && same_gains && hidden % 4 == 0 && hidden <= 4 * 256 * 16 && (!delta || partial_stride % 4 == 0) &&
      reinterpret_cast<uintptr_t>(delta) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(gain) % 16 == 0 && reinterpret_cast<uintptr_t>(post_gain) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(post_scale) % 16 == 0) {
    // which shape runs depends on the number of rows; what it computes does not: a row's sums are block
    // sums of per-thread sums either way, and the two shapes differ in how the elements are dealt to threads
    const int quads = hidden / 4;
    const bool few = n <= 128 && quads > 256;  // a decode step: spread each row over more threads
#define PYRE_LNV(THREADS, ITEMS)                                                                                       \
  hipLaunchKernelGGL((add_layernorm_vec_kernel<TD, TG, TO, THREADS, ITEMS>), dim3(n), dim3(THREADS), 0, stream, resid, \
                     static_cast<const TD*>(delta), n_partials, static_cast<size_t>(partial_stride),                   \
                     static_cast<const TG*>(post_gain), static_cast<const TG*>(post_scale), post_eps,                  \
                     static_cast<const TG*>(gain), static_cast<TO*>(out), rows, hidden, eps)
    PYRE_DISPATCH(delta ? delta_dt : kF32, TD, PYRE_DISPATCH(gain_dt, TG, PYRE_DISPATCH(out_dt, TO, {
      if (few && quads <= 1024) PYRE_LNV(1024, 1);
      else if (few) PYRE_LNV(1024, 4);
      else if (quads <= 256) PYRE_LNV(256, 1);
      else if (quads <= 1024) PYRE_LNV(256, 4);
      else PYRE_LNV(256, 16);
    })));
#undef PYRE_LNV
    return check_launch("add_layernorm");
  }
#define PYRE_LN(ITEMS)                                                                                              \
  hipLaunchKernelGGL(add_layernorm_kernel<ITEMS>, dim3(n), dim3(kThreads), 0, stream, resid, delta, delta_dt,       \
                     n_partials, static_cast<size_t>(partial_stride), bias, bias_dt, post_gain, post_gain_dt,       \
                     post_scale, post_scale_dt, post_eps, gain, gain_dt, out, out_dt, rows, hidden, eps)
  if (hidden <= 2 * kThreads) PYRE_LN(2);
  else if (hidden <= 8 * kThreads) PYRE_LN(8);
  else if (hidden <= 32 * kThreads) PYRE_LN(32);
  else PYRE_LN(64);
#undef PYRE_LN
  return check_launch("add_layernorm");
}

extern "C" int pyre_clipped_glu(const void* gu, int gu_dt, int n_partials, long partial_stride, void* out, int out_dt,
                                int n, int inter, float limit, float slope, float shift, float cubic,
                                hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(gu_dt) && known_dtype(out_dt), "clipped_glu: unknown dtype");
  PYRE_REQUIRE(n_partials >= 1 && inter > 0, "clipped_glu: bad sizes");
  if (n <= 0) return 0;
  if (gu_dt == kBF16 && out_dt == kBF16 && n_partials == 1 && inter % 8 == 0 && n > 128 &&
      reinterpret_cast<uintptr_t>(gu) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const size_t total8 = static_cast<size_t>(n) * (inter / 8);
    hipLaunchKernelGGL(clipped_glu_stream_kernel, dim3((total8 + 255) / 256), dim3(256), 0, stream,
                       static_cast<const bf16*>(gu), static_cast<bf16*>(out), total8, inter, limit, slope, shift, cubic);
    return check_launch("clipped_glu");
  }
  if (inter % 4 == 0 && partial_stride % 4 == 0 && reinterpret_cast<uintptr_t>(gu) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const size_t total4 = static_cast<size_t>(n) * (inter / 4);
    PYRE_DISPATCH(gu_dt, TI, PYRE_DISPATCH(out_dt, TO,
        hipLaunchKernelGGL((clipped_glu_vec_kernel<TI, TO>), dim3((total4 + 255) / 256), dim3(256), 0, stream,
                           static_cast<const TI*>(gu), n_partials, static_cast<size_t>(partial_stride),
                           static_cast<TO*>(out), total4, inter, limit, slope, shift, cubic)));
    return check_launch("clipped_glu");
  }
  const size_t total = static_cast<size_t>(n) * inter;
  hipLaunchKernelGGL(clipped_glu_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, gu, gu_dt, n_partials,
                     static_cast<size_t>(partial_stride), out, out_dt, total, inter, limit, slope, shift, cubic);
  return check_launch("clipped_glu");
}

extern "C" int pyre_scale(float* x, long total, float s, hipStream_t stream) {
  if (total <= 0) return 0;
  hipLaunchKernelGGL(scale_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, x, static_cast<size_t>(total), s);
  return check_launch("scale");
}
