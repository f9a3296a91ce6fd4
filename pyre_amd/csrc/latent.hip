// What stands between the input product and the attention kernels of two mixers that keep less than a
// key and a value per head and token, and the small per-head products of the second:
//
//   rope_tied_write  attention whose values are its keys as projected: sums the product's partial sums,
//                    adds the bias, turns the first `rot` elements of every query and key head by position
//                    (element e with e + rot/2), stores the queries, the turned keys as keys and the keys
//                    as they were before turning as values (k, v [pages, nkv, page, d]).
//   latent_write     attention over one compressed row per token: stores the queries and, if the layer
//                    makes the row itself, the row divided by its root mean square, times a gain
//                    (c [pages, 1, page, rank]).
//   head_matmul      out[n, h, :] = x[n, h, :] W[h] for every head h, W [heads, din, dout]: the products
//                    that carry a query into the compressed row's space and a weighted row out of it.
//
// All arithmetic is float32; roundings happen at the stores of 16-bit outputs only.
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

constexpr int kThreads = 256;

struct Proj {
  const void* data;
  int dt, count;
  size_t stride;
  int ld, col0;
  const void* bias;
  int bias_dt;
};

__device__ inline float proj_at(const Proj& p, int n, int col) {
  const size_t at = static_cast<size_t>(n) * p.ld + p.col0 + col;
  float v = 0.f;
  for (int i = 0; i < p.count; ++i) v += load_as_float(p.data, p.dt, i * p.stride + at);
  if (p.bias) v += load_as_float(p.bias, p.bias_dt, col);
  return v;
}

template <typename TC>
__global__ __launch_bounds__(kThreads) void rope_tied_write_kernel(Proj proj, void* __restrict__ q_out, int q_dt,
                                                                   TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                                                   const float* __restrict__ cos_t,
                                                                   const float* __restrict__ sin_t, int rot,
                                                                   const int* __restrict__ positions,
                                                                   const int* __restrict__ slots, int nq, int nkv, int d,
                                                                   int page_size, int write_kv) {
  const int n = blockIdx.x, half = rot / 2;
  const int pos = positions[n];
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  for (int i = threadIdx.x; i < (nq + nkv) * d; i += kThreads) {
    const int head = i / d, e = i % d;
    const float x = proj_at(proj, n, i);
    float turned = x;
    if (e < rot) {
      const int j = e < half ? e : e - half;
      const float c = cos_t[static_cast<size_t>(pos) * half + j], s = sin_t[static_cast<size_t>(pos) * half + j];
      const float y = proj_at(proj, n, head * d + (e < half ? e + half : e - half));
      float a, b;
      if (e < half) {
        rotate_pair(x, y, c, s, a, b);
        turned = a;
      } else {
        rotate_pair(y, x, c, s, a, b);
        turned = b;
      }
    }
    if (head < nq) {
      store_from_float(q_out, q_dt, static_cast<size_t>(n) * nq * d + i, turned);
    } else if (slot >= 0) {
      const size_t at = ((static_cast<size_t>(page) * nkv + (head - nq)) * page_size + off) * d + e;
      k_cache[at] = from_float<TC>(turned);
      v_cache[at] = from_float<TC>(x);
    }
  }
}

template <typename TC>
__global__ __launch_bounds__(kThreads) void latent_write_kernel(Proj proj, void* __restrict__ q_out, int q_dt,
                                                                TC* __restrict__ c_cache, const void* __restrict__ gain,
                                                                int gain_dt, float eps, const int* __restrict__ slots,
                                                                int q_width, int rank, int page_size, int write) {
  __shared__ float scratch[16];
  const int n = blockIdx.x;
  for (int i = threadIdx.x; i < q_width; i += kThreads)
    store_from_float(q_out, q_dt, static_cast<size_t>(n) * q_width + i, proj_at(proj, n, i));
  if (!write) return;
  const int slot = slots[n];
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += kThreads) {
    const float v = proj_at(proj, n, q_width + i);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  if (slot < 0) return;
  const float inv = 1.f / sqrtf(ss / static_cast<float>(rank) + eps);
  TC* dst = c_cache + static_cast<size_t>(slot) * rank;  // pages of [1, page, rank]: slot = page * page_size + offset
  for (int i = threadIdx.x; i < rank; i += kThreads)
    dst[i] = from_float<TC>(proj_at(proj, n, q_width + i) * inv * load_as_float(gain, gain_dt, i));
}

// A block: kRows tokens of one head against all of W[h]. Thread c makes column c (+ 256, ...) of every token.
constexpr int kRows = 16;
template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(kThreads) void head_matmul_kernel(const TX* __restrict__ x, int x_ld, const TW* __restrict__ w,
                                                               TO* __restrict__ out, int out_ld, int n, int din, int dout) {
  extern __shared__ float xs[];  // [kRows][din]
  const int h = blockIdx.y, n0 = blockIdx.x * kRows, rows = min(kRows, n - n0);
  for (int i = threadIdx.x; i < kRows * din; i += kThreads) {
    const int r = i / din, e = i % din;
    xs[i] = r < rows ? to_float(x[static_cast<size_t>(n0 + r) * x_ld + h * din + e]) : 0.f;
  }
  __syncthreads();
  const TW* wh = w + static_cast<size_t>(h) * din * dout;
  for (int c = threadIdx.x; c < dout; c += kThreads) {
    float acc[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) acc[r] = 0.f;
    for (int e = 0; e < din; ++e) {
      const float wv = to_float(wh[static_cast<size_t>(e) * dout + c]);
#pragma unroll
      for (int r = 0; r < kRows; ++r) acc[r] = fmaf(xs[r * din + e], wv, acc[r]);
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r)
      if (r < rows) out[static_cast<size_t>(n0 + r) * out_ld + h * dout + c] = from_float<TO>(acc[r]);
  }
}

}  // namespace

extern "C" int pyre_rope_tied_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                                    const void* bias, int bias_dt, void* q_out, int q_dt, void* k_cache, void* v_cache,
                                    int cache_dt, const float* cos_t, const float* sin_t, int rot, const int* positions,
                                    const int* slots, int n, int nq, int nkv, int d, int page_size, int write_kv,
                                    hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(proj_dt) && known_dtype(q_dt) && known_dtype(cache_dt) && n_partials >= 1, "rope_tied_write: bad dtypes");
  PYRE_REQUIRE(!bias || known_dtype(bias_dt), "rope_tied_write: unknown bias dtype");
  PYRE_REQUIRE(nq > 0 && nkv > 0 && d > 0 && page_size > 0, "rope_tied_write: bad geometry");
  PYRE_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0 && (rot == 0 || (cos_t && sin_t)), "rope_tied_write: %d turned elements do not fit a head of %d", rot, d);
  PYRE_REQUIRE(!write_kv || (k_cache && v_cache && slots), "rope_tied_write: a cache write needs caches and slots");
  if (n <= 0) return 0;
  const Proj p{proj, proj_dt, n_partials, static_cast<size_t>(partial_stride), ld, col0, bias, bias_dt};
  PYRE_DISPATCH(cache_dt, TC,
      hipLaunchKernelGGL(rope_tied_write_kernel<TC>, dim3(n), dim3(kThreads), 0, stream, p, q_out, q_dt,
                         static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), cos_t, sin_t, rot, positions, slots, nq,
                         nkv, d, page_size, write_kv));
  return check_launch("rope_tied_write");
}

extern "C" int pyre_latent_write(const void* proj, int proj_dt, int n_partials, long partial_stride, int ld, int col0,
                                 void* q_out, int q_dt, void* c_cache, int cache_dt, const void* gain, int gain_dt,
                                 float eps, const int* slots, int n, int q_width, int rank, int page_size, int write,
                                 hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(proj_dt) && known_dtype(q_dt) && known_dtype(cache_dt) && n_partials >= 1, "latent_write: bad dtypes");
  PYRE_REQUIRE(q_width > 0 && rank > 0 && page_size > 0, "latent_write: bad geometry");
  PYRE_REQUIRE(!write || (c_cache && gain && slots && known_dtype(gain_dt) && eps > 0.f), "latent_write: a cache write needs cache, gain, slots and eps");
  if (n <= 0) return 0;
  const Proj p{proj, proj_dt, n_partials, static_cast<size_t>(partial_stride), ld, col0, nullptr, 0};
  PYRE_DISPATCH(cache_dt, TC,
      hipLaunchKernelGGL(latent_write_kernel<TC>, dim3(n), dim3(kThreads), 0, stream, p, q_out, q_dt,
                         static_cast<TC*>(c_cache), gain, gain_dt, eps, slots, q_width, rank, page_size, write));
  return check_launch("latent_write");
}

extern "C" int pyre_head_matmul(const void* x, int x_ld, const void* w, void* out, int out_ld, int dt, int n, int heads,
                                int din, int dout, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(dt), "head_matmul: unknown dtype");
  PYRE_REQUIRE(heads > 0 && heads <= 65535 && din > 0 && dout > 0 && x_ld >= heads * din && out_ld >= heads * dout,
               "head_matmul: bad geometry");
  PYRE_REQUIRE(static_cast<size_t>(kRows) * din * sizeof(float) <= 64 * 1024, "head_matmul: heads of %d elements are too wide", din);
  if (n <= 0) return 0;
  const dim3 grid((n + kRows - 1) / kRows, heads);
  const size_t lds = sizeof(float) * kRows * din;
  PYRE_DISPATCH(dt, T,
      hipLaunchKernelGGL((head_matmul_kernel<T, T, T>), grid, dim3(kThreads), lds, stream, static_cast<const T*>(x), x_ld,
                         static_cast<const T*>(w), static_cast<T*>(out), out_ld, n, din, dout));
  return check_launch("head_matmul");
}
