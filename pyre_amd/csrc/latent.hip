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
#include "pyre_vec4.h"

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

// The same with a wave per token and head, four elements a lane and an element's partial sums asked for together:
// head sizes, the number of turned elements of each half, the product's width, first column and stride are multiples
// of four; queries, caches and bias share one element type.
template <typename TP, typename TC>
__global__ __launch_bounds__(kWave) void rope_tied_write_vec_kernel(const TP* __restrict__ proj, int count, size_t stride,
                                                                    int ld, int col0, const TC* __restrict__ bias,
                                                                    TC* __restrict__ q_out, TC* __restrict__ k_cache,
                                                                    TC* __restrict__ v_cache, const float* __restrict__ cos_t,
                                                                    const float* __restrict__ sin_t, int rot,
                                                                    const int* __restrict__ positions,
                                                                    const int* __restrict__ slots, int nq, int nkv, int d,
                                                                    int page_size, int write_kv) {
  __shared__ __attribute__((aligned(16))) float xs[4 * kWave];
  const int n = blockIdx.x, head = blockIdx.y, e = 4 * threadIdx.x, half = rot / 2;
  float4 x = {0.f, 0.f, 0.f, 0.f};
  if (e < d) {
    x = sum_partials4(proj + static_cast<size_t>(n) * ld + col0 + head * d + e, stride, count);
    if (bias) x = add4(x, Vec4<TC>::load(bias + head * d + e));
    *reinterpret_cast<float4*>(xs + e) = x;
  }
  __syncthreads();
  if (e >= d) return;
  float4 t = x;
  if (e < rot) {  // the four elements lie in the same half, their partners in the other
    const bool low = e < half;
    const int j = low ? e : e - half;
    const float4 y = *reinterpret_cast<const float4*>(xs + (low ? e + half : e - half));
    const size_t at = static_cast<size_t>(positions[n]) * half + j;
    const float4 c = *reinterpret_cast<const float4*>(cos_t + at), sn = *reinterpret_cast<const float4*>(sin_t + at);
    float a, b;
    if (low) {
      rotate_pair(x.x, y.x, c.x, sn.x, a, b), t.x = a;
      rotate_pair(x.y, y.y, c.y, sn.y, a, b), t.y = a;
      rotate_pair(x.z, y.z, c.z, sn.z, a, b), t.z = a;
      rotate_pair(x.w, y.w, c.w, sn.w, a, b), t.w = a;
    } else {
      rotate_pair(y.x, x.x, c.x, sn.x, a, b), t.x = b;
      rotate_pair(y.y, x.y, c.y, sn.y, a, b), t.y = b;
      rotate_pair(y.z, x.z, c.z, sn.z, a, b), t.z = b;
      rotate_pair(y.w, x.w, c.w, sn.w, a, b), t.w = b;
    }
  }
  if (head < nq) {
    Vec4<TC>::store(q_out + (static_cast<size_t>(n) * nq + head) * d + e, t);
    return;
  }
  const int slot = write_kv ? slots[n] : -1;
  if (slot < 0) return;
  const size_t at = ((static_cast<size_t>(slot / page_size) * nkv + (head - nq)) * page_size + slot % page_size) * d + e;
  Vec4<TC>::store(k_cache + at, t);
  Vec4<TC>::store(v_cache + at, x);
}

// Block (n, 0) norms and stores the compressed row, blocks (n, 1 ...) pass 1,024 query columns each: four elements a
// thread (all widths, first column and strides are multiples of four; gain and cache share one element type).
template <typename TP, typename TC>
__global__ __launch_bounds__(kThreads) void latent_write_vec_kernel(const TP* __restrict__ proj, int count, size_t stride, int ld,
                                                                    int col0, TC* __restrict__ q_out, TC* __restrict__ c_cache,
                                                                    const TC* __restrict__ gain, float eps,
                                                                    const int* __restrict__ slots, int q_width, int rank,
                                                                    int write) {
  __shared__ float scratch[16];
  const int n = blockIdx.x, e = 4 * threadIdx.x;
  const TP* in = proj + static_cast<size_t>(n) * ld + col0;
  if (blockIdx.y > 0) {
    const int c = (blockIdx.y - 1) * 4 * kThreads + e;
    if (c < q_width) Vec4<TC>::store(q_out + static_cast<size_t>(n) * q_width + c, sum_partials4(in + c, stride, count));
    return;
  }
  if (!write) return;
  float4 v = {0.f, 0.f, 0.f, 0.f};
  if (e < rank) v = sum_partials4(in + q_width + e, stride, count);
  const float ss = block_sum((v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w), scratch);
  const int slot = slots[n];
  if (slot < 0 || e >= rank) return;
  const float inv = 1.f / sqrtf(ss / static_cast<float>(rank) + eps);
  const float4 g = Vec4<TC>::load(gain + e);
  Vec4<TC>::store(c_cache + static_cast<size_t>(slot) * rank + e, float4{v.x * inv * g.x, v.y * inv * g.y, v.z * inv * g.z, v.w * inv * g.w});
}

// A block: kRows tokens of one head against 64 columns of W[h]. Thread (c, part) walks a quarter of the head's
// elements for column c of every token; the four parts are added through LDS in their order.
constexpr int kRows = 16;
constexpr int kCols = 64;
template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(kThreads) void head_matmul_kernel(const TX* __restrict__ x, int x_ld, const TW* __restrict__ w,
                                                               TO* __restrict__ out, int out_ld, int n, int din, int dout) {
  extern __shared__ float lds[];  // xs [kRows][din], then sums [3][kRows][kCols]
  float* xs = lds;
  float* sums = lds + kRows * din;
  const int h = blockIdx.y, n0 = blockIdx.x * kRows, rows = min(kRows, n - n0);
  const int c = threadIdx.x % kCols, part = threadIdx.x / kCols, col = blockIdx.z * kCols + c;
  for (int i = threadIdx.x; i < kRows * din; i += kThreads) {
    const int r = i / din, e = i % din;
    xs[i] = r < rows ? to_float(x[static_cast<size_t>(n0 + r) * x_ld + h * din + e]) : 0.f;
  }
  __syncthreads();
  const int per = (din + 3) / 4, e0 = part * per, e1 = min(din, e0 + per);
  const TW* wh = w + static_cast<size_t>(h) * din * dout + min(col, dout - 1);
  float acc[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) acc[r] = 0.f;
  int e = e0;
  for (; e + 8 <= e1; e += 8) {  // eight of W's rows on their way together
    float wv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) wv[u] = to_float(wh[static_cast<size_t>(e + u) * dout]);
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int r = 0; r < kRows; ++r) acc[r] = fmaf(xs[r * din + e + u], wv[u], acc[r]);
  }
  for (; e < e1; ++e) {
    const float wv = to_float(wh[static_cast<size_t>(e) * dout]);
#pragma unroll
    for (int r = 0; r < kRows; ++r) acc[r] = fmaf(xs[r * din + e], wv, acc[r]);
  }
  if (part > 0)
#pragma unroll
    for (int r = 0; r < kRows; ++r) sums[((part - 1) * kRows + r) * kCols + c] = acc[r];
  __syncthreads();
  if (part > 0 || col >= dout) return;
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const float total = ((acc[r] + sums[r * kCols + c]) + sums[(kRows + r) * kCols + c]) + sums[(2 * kRows + r) * kCols + c];
    if (r < rows) out[static_cast<size_t>(n0 + r) * out_ld + h * dout + col] = from_float<TO>(total);
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
  const auto a16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  if (d % 4 == 0 && d <= 4 * kWave && rot % 8 == 0 && ld % 4 == 0 && col0 % 4 == 0 && partial_stride % 4 == 0 && q_dt == cache_dt &&
      (!bias || bias_dt == cache_dt) && nq + nkv <= 65535 && a16(proj) && a16(bias) && a16(q_out) && a16(k_cache) && a16(v_cache) &&
      a16(cos_t) && a16(sin_t)) {
    PYRE_DISPATCH(proj_dt, TP, PYRE_DISPATCH(cache_dt, TC,
        hipLaunchKernelGGL((rope_tied_write_vec_kernel<TP, TC>), dim3(n, nq + nkv), dim3(kWave), 0, stream,
                           static_cast<const TP*>(proj), n_partials, static_cast<size_t>(partial_stride), ld, col0,
                           static_cast<const TC*>(bias), static_cast<TC*>(q_out), static_cast<TC*>(k_cache),
                           static_cast<TC*>(v_cache), cos_t, sin_t, rot, positions, slots, nq, nkv, d, page_size, write_kv)));
    return check_launch("rope_tied_write");
  }
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
  const auto a16 = [](const void* q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  if (q_width % 4 == 0 && rank % 4 == 0 && rank <= 4 * kThreads && ld % 4 == 0 && col0 % 4 == 0 && partial_stride % 4 == 0 &&
      q_dt == cache_dt && (!write || gain_dt == cache_dt) && a16(proj) && a16(q_out) && a16(c_cache) && a16(gain)) {
    const dim3 grid(n, 1 + (q_width + 4 * kThreads - 1) / (4 * kThreads));
    PYRE_DISPATCH(proj_dt, TP, PYRE_DISPATCH(cache_dt, TC,
        hipLaunchKernelGGL((latent_write_vec_kernel<TP, TC>), grid, dim3(kThreads), 0, stream, static_cast<const TP*>(proj),
                           n_partials, static_cast<size_t>(partial_stride), ld, col0, static_cast<TC*>(q_out),
                           static_cast<TC*>(c_cache), static_cast<const TC*>(gain), eps, slots, q_width, rank, write)));
    return check_launch("latent_write");
  }
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
  const size_t lds = sizeof(float) * (static_cast<size_t>(kRows) * din + 3 * kRows * kCols);
  PYRE_REQUIRE(lds <= 64 * 1024 && (dout + kCols - 1) / kCols <= 65535, "head_matmul: heads of %d elements are too wide", din);
  if (n <= 0) return 0;
  const dim3 grid((n + kRows - 1) / kRows, heads, (dout + kCols - 1) / kCols);
  PYRE_DISPATCH(dt, T,
      hipLaunchKernelGGL((head_matmul_kernel<T, T, T>), grid, dim3(kThreads), lds, stream, static_cast<const T*>(x), x_ld,
                         static_cast<const T*>(w), static_cast<T*>(out), out_ld, n, din, dout));
  return check_launch("head_matmul");
}
