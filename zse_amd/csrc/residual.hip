// Joining two sublayers that read the same norm to the float residual stream:
//
//   h <- h + (a + b + bias);    out = h / sqrt(mean(h^2) + eps) * gain     (if a next norm is given)
//
// a and b are each either activations [T, W] (parts = 0) or ``parts`` float planes [parts, T, W]
// that are added up in order (partial sums of a product that split K, or the results of
// several paths of one sublayer); either may be absent.  The sum of the sublayers is formed
// first and then added to the stream, all in float.  One block per row.
#include "common.h"
#include "packed_call.h"

extern "C" int zk_steplist_register(const char* name, int nargs, void* fn);
#define ZK_ENTER(fn) \
  static const int fn##_entered = zk_steplist_register(#fn, zk_packed::Call<fn>::nargs, (void*)zk_packed::Call<fn>::call);

__device__ __forceinline__ float planes_value(const void* __restrict__ p, int parts, size_t plane, size_t at) {
  if (p == nullptr) return 0.f;
  if (parts <= 0) return to_f32(((const act_t*)p)[at]);
  float x = ((const float*)p)[at];
  for (int i = 1; i < parts; i++) x += ((const float*)p)[i * plane + at];
  return x;
}

__global__ void sum_norm_kernel(float* __restrict__ h, const void* __restrict__ a, int a_parts,
                                const void* __restrict__ b, int b_parts, const float* __restrict__ bias,
                                const float* __restrict__ w_next, float eps, int unit_offset, act_t* __restrict__ out,
                                int W) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t plane = (size_t)gridDim.x * W, row = (size_t)r * W;
  float* hr = h + row;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float y = planes_value(a, a_parts, plane, row + i) + planes_value(b, b_parts, plane, row + i);
    if (bias) y += bias[i];
    const float v = hr[i] + y;
    hr[i] = v;
    ss = fmaf(v, v, ss);
  }
  if (!w_next) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)      // each thread re-reads what it wrote
    out[row + i] = from_f32<act_t>(hr[i] * inv * (unit_offset ? 1.0f + w_next[i] : w_next[i]));
}

// y[t, :] += bias
__global__ void add_bias_kernel(act_t* __restrict__ y, const float* __restrict__ bias, int W) {
  const size_t row = (size_t)blockIdx.x * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) y[row + i] = from_f32<act_t>(to_f32(y[row + i]) + bias[i]);
}

// out[t, :] = sum of float planes, rounded once
__global__ void planes_sum_kernel(const float* __restrict__ p, int parts, act_t* __restrict__ out, int W) {
  const size_t plane = (size_t)gridDim.x * W, row = (size_t)blockIdx.x * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) out[row + i] = from_f32<act_t>(planes_value(p, parts, plane, row + i));
}

extern "C" {

int zk_sum_norm(float* h, const void* a, int a_parts, const void* b, int b_parts, const float* bias, const float* w_next,
                float eps, int unit_offset, void* out, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && a_parts >= 0 && b_parts >= 0, "zk_sum_norm: bad sizes");
  ZK_REQUIRE(w_next == nullptr || out != nullptr, "zk_sum_norm: a next norm without output");
  if (T == 0) return 0;
  // in the 32-bit library the block is always 256 wide: the order of a row's sums must not follow
  // from how many rows a step brings
  const int threads = (ZSE_ACT_BF16 && T <= 64 && W >= 1024) ? 1024 : 256;
  sum_norm_kernel<<<T, threads, 0, (hipStream_t)stream>>>(h, a, a_parts, b, b_parts, bias, w_next, eps, unit_offset,
                                                         (act_t*)out, W);
  return zk_launch_status("zk_sum_norm");
}

int zk_add_bias(void* y, const float* bias, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && bias != nullptr, "zk_add_bias: bad sizes");
  if (T == 0) return 0;
  add_bias_kernel<<<T, 256, 0, (hipStream_t)stream>>>((act_t*)y, bias, W);
  return zk_launch_status("zk_add_bias");
}

int zk_planes_sum(const float* planes, int parts, void* out, int T, int W, void* stream) {
  ZK_REQUIRE(T >= 0 && W > 0 && parts >= 1, "zk_planes_sum: bad sizes");
  if (T == 0) return 0;
  planes_sum_kernel<<<T, 256, 0, (hipStream_t)stream>>>(planes, parts, (act_t*)out, W);
  return zk_launch_status("zk_planes_sum");
}

}  // extern "C"

ZK_ENTER(zk_sum_norm)
ZK_ENTER(zk_add_bias)
ZK_ENTER(zk_planes_sum)
