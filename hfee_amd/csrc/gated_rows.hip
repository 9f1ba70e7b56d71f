// Row-wise steps around sub-layers whose results pass a gate before they are normed and added:
//
//   add_table_rows:   x[r] += table[index[r]]                 (a learned vector a position, added to the lookup)
//   gated_norm_add:   v = (a y[r] + b y2[r]) * sigmoid(g[r] + c);  x[r] += v / sqrt(mean(v^2) + eps) * w,
//                     and, if asked, in the same launch the norm of the new row for the sub-layer that
//                     follows: next[r] = x[r] / sqrt(mean(x[r]^2) + eps2) * w2.
//                     y2 (a second mixer beside the first), the gate g with its bias c: each optional.
//   scaled_add:       x += a y + b y2
//
// All sums in float32, one workgroup a row, a fixed order of additions (which depends on the row's width and
// alignment only, never on the other rows of the step).
#include "common.h"

using namespace hfee;

namespace {

template <typename T>
__global__ __launch_bounds__(256) void add_table_rows_kernel(float* __restrict__ x, int d, const T* __restrict__ table,
                                                             const int* __restrict__ index) {
  const int64_t r = blockIdx.x;
  const T* row = table + (int64_t)index[r] * d;
  for (int j = blockIdx.y * blockDim.x + threadIdx.x; j < d; j += gridDim.y * blockDim.x) x[r * d + j] += to_float<T>(row[j]);
}

template <typename TG>
__device__ __forceinline__ float gated_value(const float* y, const float* y2, float a, float b, const TG* g,
                                             const float* gate_bias, int j) {
  float v = y2 != nullptr ? fmaf(a, y[j], b * y2[j]) : a * y[j];
  if (g != nullptr) v *= 1.0f / (1.0f + expf(-(to_float<TG>(g[j]) + (gate_bias != nullptr ? gate_bias[j] : 0.f))));
  return v;
}

template <typename TG, typename TN>
__global__ __launch_bounds__(256) void gated_norm_add_kernel(
    float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ y2, float a, float b,
    const TG* __restrict__ gate, int64_t ldg, const float* __restrict__ gate_bias, const float* __restrict__ w, float eps,
    TN* __restrict__ next, const float* __restrict__ w2, float eps2, int d) {
  __shared__ float scratch[16];
  const int64_t r = blockIdx.x;
  const float* yr = y + r * d;
  const float* y2r = y2 != nullptr ? y2 + r * d : nullptr;
  const TG* gr = gate != nullptr ? gate + r * ldg : nullptr;
  float* xr = x + r * d;
  float ss = 0.f;
  for (int j = threadIdx.x; j < d; j += blockDim.x) {
    const float v = gated_value<TG>(yr, y2r, a, b, gr, gate_bias, j);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  float ss2 = 0.f;
  for (int j = threadIdx.x; j < d; j += blockDim.x) {
    const float nx = xr[j] + gated_value<TG>(yr, y2r, a, b, gr, gate_bias, j) * inv * w[j];
    xr[j] = nx;
    ss2 = fmaf(nx, nx, ss2);
  }
  if (next == nullptr) return;
  ss2 = block_sum(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)d + eps2);
  TN* nr = next + r * d;
  for (int j = threadIdx.x; j < d; j += blockDim.x)      // (a thread reads back what it wrote itself)
    nr[j] = from_float<TN>(xr[j] * inv2 * w2[j]);
}


// The same for rows of up to 1024 * K values that are whole groups of four: a thread asks for all it needs of
// the row at once (K groups of four of y, y2, the gate and x), keeps the gated values in registers between the
// sum of squares and the addition, and the new row between the second sum and the following norm.  A row is
// read once, and a step of a few rows is one wait for memory instead of one a loop turn.
template <typename TG, typename TN, int K>
__global__ __launch_bounds__(256) void gated_norm_add_held_kernel(
    float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ y2, float a, float b,
    const TG* __restrict__ gate, int64_t ldg, const float* __restrict__ gate_bias, const float* __restrict__ w, float eps,
    TN* __restrict__ next, const float* __restrict__ w2, float eps2, int d) {
  __shared__ float scratch[16];
  const int64_t r = blockIdx.x;
  float v[K][4], xs[K][4], ws[K][4];
  {
    float second[K][4], g[K][4], gb[K][4];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int j = (k * 256 + threadIdx.x) * 4;
      const bool in = j < d;
      const int jj = in ? j : 0;
      load4<float>(v[k], y + r * d + jj);
      load4<float>(xs[k], x + r * d + jj);
      load4<float>(ws[k], w + jj);
      if (y2 != nullptr) load4<float>(second[k], y2 + r * d + jj);
      if (gate != nullptr) load4<TG>(g[k], gate + r * ldg + jj);
      if (gate_bias != nullptr) load4<float>(gb[k], gate_bias + jj);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float t = y2 != nullptr ? fmaf(a, v[k][i], b * second[k][i]) : a * v[k][i];
        if (gate != nullptr) t *= 1.0f / (1.0f + expf(-(g[k][i] + (gate_bias != nullptr ? gb[k][i] : 0.f))));
        v[k][i] = in ? t : 0.f;
      }
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k)
#pragma unroll
    for (int i = 0; i < 4; ++i) ss = fmaf(v[k][i], v[k][i], ss);
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int j = (k * 256 + threadIdx.x) * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xs[k][i] = j < d ? xs[k][i] + v[k][i] * inv * ws[k][i] : 0.f;
      ss2 = fmaf(xs[k][i], xs[k][i], ss2);
    }
    if (j < d) store4<float>(x + r * d + j, xs[k]);
  }
  if (next == nullptr) return;
  ss2 = block_sum(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)d + eps2);
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int j = (k * 256 + threadIdx.x) * 4;
    if (j >= d) continue;
    load4<float>(ws[k], w2 + j);
#pragma unroll
    for (int i = 0; i < 4; ++i) xs[k][i] = xs[k][i] * inv2 * ws[k][i];
    store4<TN>(next + r * d + j, xs[k]);
  }
}

}  // namespace

HFEE_API int hfee_add_table_rows(float* x, int n, int d, const void* table, int dtype, const int* index, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && d > 0 && table != nullptr && index != nullptr, "add_table_rows: bad arguments");
  if (n == 0) return 0;
  int parts = (d + 1023) / 1024;
  if (parts > 64) parts = 64;
  if (dtype == 0) add_table_rows_kernel<float><<<dim3(n, parts), 256, 0, stream>>>(x, d, (const float*)table, index);
  else if (dtype == 1) add_table_rows_kernel<bf16_t><<<dim3(n, parts), 256, 0, stream>>>(x, d, (const bf16_t*)table, index);
  else return fail("add_table_rows: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("add_table_rows");
  return 0;
}

// gate_dtype / next_dtype: 0 float32, 1 bfloat16.  y, y2: float32 [n, d]; w, w2, gate_bias: float32 [d].
HFEE_API int hfee_gated_norm_add(float* x, const float* y, const float* y2, float a, float b, const void* gate,
                                 int gate_dtype, int64_t ldg, const float* gate_bias, const float* w, float eps,
                                 void* next, int next_dtype, const float* w2, float eps2, int n, int d, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && d > 0 && y != nullptr && w != nullptr, "gated_norm_add: bad sizes n=%d d=%d", n, d);
  HFEE_REQUIRE(eps >= 0.f && eps2 >= 0.f, "gated_norm_add: eps must not be negative");
  HFEE_REQUIRE(next == nullptr || w2 != nullptr, "gated_norm_add: the following norm needs its weight");
  HFEE_REQUIRE(gate == nullptr || ldg >= d, "gated_norm_add: the gate's rows are too short");
  if (n == 0) return 0;
  const auto aligned = [](const void* p, int to) { return (reinterpret_cast<uintptr_t>(p) & (uintptr_t)(to - 1)) == 0; };
  const bool held = d % 4 == 0 && d <= 8192 && aligned(x, 16) && aligned(y, 16) && aligned(y2, 16) && aligned(w, 16) &&
                    aligned(gate_bias, 16) && aligned(w2, 16) && aligned(next, 16) &&
                    (gate == nullptr || (ldg % 4 == 0 && aligned(gate, 16)));
  const int code = (gate_dtype & 1) | ((next_dtype & 1) << 1);
#define LAUNCH(TG, TN)                                                                                               \
  do {                                                                                                               \
    if (!held)                                                                                                       \
      gated_norm_add_kernel<TG, TN><<<n, 256, 0, stream>>>(x, y, y2, a, b, (const TG*)gate, ldg, gate_bias, w, eps,  \
                                                           (TN*)next, w2, eps2, d);                                  \
    else if (d <= 1024)                                                                                              \
      gated_norm_add_held_kernel<TG, TN, 1><<<n, 256, 0, stream>>>(x, y, y2, a, b, (const TG*)gate, ldg, gate_bias,  \
                                                                   w, eps, (TN*)next, w2, eps2, d);                  \
    else if (d <= 2048)                                                                                              \
      gated_norm_add_held_kernel<TG, TN, 2><<<n, 256, 0, stream>>>(x, y, y2, a, b, (const TG*)gate, ldg, gate_bias,  \
                                                                   w, eps, (TN*)next, w2, eps2, d);                  \
    else if (d <= 4096)                                                                                              \
      gated_norm_add_held_kernel<TG, TN, 4><<<n, 256, 0, stream>>>(x, y, y2, a, b, (const TG*)gate, ldg, gate_bias,  \
                                                                   w, eps, (TN*)next, w2, eps2, d);                  \
    else                                                                                                             \
      gated_norm_add_held_kernel<TG, TN, 8><<<n, 256, 0, stream>>>(x, y, y2, a, b, (const TG*)gate, ldg, gate_bias,  \
                                                                   w, eps, (TN*)next, w2, eps2, d);                  \
  } while (0)
  if (code == 0) LAUNCH(float, float);
  else if (code == 1) LAUNCH(bf16_t, float);
  else if (code == 2) LAUNCH(float, bf16_t);
  else LAUNCH(bf16_t, bf16_t);
#undef LAUNCH
  HFEE_CHECK_LAUNCH("gated_norm_add");
  return 0;
}

namespace {
__global__ __launch_bounds__(256) void scaled_add_kernel(float* __restrict__ x, const float* __restrict__ y, float a,
                                                         const float* __restrict__ y2, float b, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) x[i] += y2 != nullptr ? fmaf(a, y[i], b * y2[i]) : a * y[i];
}
}  // namespace

// x += a y + b y2 (y2 optional), all float32 and contiguous.
HFEE_API int hfee_scaled_add(float* x, const float* y, float a, const float* y2, float b, int64_t count, hipStream_t stream) {
  HFEE_REQUIRE(count >= 0 && (count + 255) / 256 <= 0x7fffffff && y != nullptr, "scaled_add: bad sizes");
  if (count == 0) return 0;
  scaled_add_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(x, y, a, y2, b, count);
  HFEE_CHECK_LAUNCH("scaled_add");
  return 0;
}

namespace {
// A workgroup a row: x += a y, then next = x / sqrt(mean(x^2) + eps) * w in the engine's dtype (the norm of
// whatever reads the stream next).  A thread keeps its elements of the new row in registers between the sum
// and the scaling where it has at most 16 of them; a longer row is read again.  256 threads a row, 1,024
// where the rows are few (a row's time is then the chain of its loads).
constexpr int kAddNormKeep = 16;

template <typename T>
__global__ __launch_bounds__(1024) void scaled_add_norm_kernel(float* __restrict__ x, const float* __restrict__ y, float a,
                                                              T* __restrict__ next, const float* __restrict__ w, float eps,
                                                              int width) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float* xr = x + row * width;
  const float* yr = y + row * width;
  T* nr = next + row * width;
  float kept[kAddNormKeep];
  float ss = 0.f;
  int i = 0;
  for (int c = threadIdx.x; c < width; c += blockDim.x, ++i) {
    const float v = fmaf(a, yr[c], xr[c]);
    xr[c] = v;
    if (i < kAddNormKeep) kept[i] = v;
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  i = 0;
  for (int c = threadIdx.x; c < width; c += blockDim.x, ++i) {
    const float v = i < kAddNormKeep ? kept[i] : xr[c];
    nr[c] = from_float<T>(v * inv * w[c]);
  }
}
}  // namespace

// x (float32 [n, width], contiguous) += a y; next ([n, width] in dtype) = the RMS norm of the new rows with weight w.
HFEE_API int hfee_scaled_add_norm(float* x, const float* y, float a, void* next, int dtype, const float* w, float eps, int n,
                                  int width, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && width > 0 && y != nullptr && next != nullptr && w != nullptr && eps >= 0.f, "scaled_add_norm: bad arguments");
  if (n == 0) return 0;
  const int threads = n <= 64 && width > 1024 ? 1024 : 256;
  if (dtype == 0) scaled_add_norm_kernel<float><<<n, threads, 0, stream>>>(x, y, a, (float*)next, w, eps, width);
  else if (dtype == 1) scaled_add_norm_kernel<bf16_t><<<n, threads, 0, stream>>>(x, y, a, (bf16_t*)next, w, eps, width);
  else return fail("scaled_add_norm: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("scaled_add_norm");
  return 0;
}
