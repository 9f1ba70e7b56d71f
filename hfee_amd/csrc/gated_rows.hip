// Row-wise steps around sub-layers whose results pass a gate before they are normed and added:
//
//   add_table_rows:   x[r] += table[index[r]]                 (a learned vector a position, added to the lookup)
//   gated_norm_add:   v = (a y[r] + b y2[r]) * sigmoid(g[r] + c);  x[r] += v / sqrt(mean(v^2) + eps) * w,
//                     and, if asked, in the same launch the norm of the new row for the sub-layer that
//                     follows: next[r] = x[r] / sqrt(mean(x[r]^2) + eps2) * w2.
//                     y2 (a second mixer beside the first), the gate g with its bias c: each optional.
//   scaled_add:       x += a y + b y2
//
// All sums in float32, one workgroup a row, a fixed order of additions.
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
#define LAUNCH(TG, TN)                                                                                               \
  gated_norm_add_kernel<TG, TN><<<n, 256, 0, stream>>>(x, y, y2, a, b, (const TG*)gate, ldg, gate_bias, w, eps,      \
                                                       (TN*)next, w2, eps2, d)
  const int code = (gate_dtype & 1) | ((next_dtype & 1) << 1);
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
