// Row-wise and element-wise kernels of layers that are not plain pre-norm attention blocks: layer norm
// with weight and bias, a per-head unit norm with gate, the xIELU and tanh activations, the weighted
// average over the outputs of all earlier layers, a scaled sum of two branches into the residual
// stream, and a scale.
//
// Acc = double is the exact path (float32 storage, float64 sums and one rounding at the end);
// otherwise sums are float. Norms, gates and averages are float arithmetic in both; only the
// results that feed a matrix product are rounded to the activation type.
#include "common.h"

namespace alofa {

// ---- layer norm ------------------------------------------------------------------------------
// y = (x - mean) / sqrt(var + eps) * w + b per row, var = mean of the squared deviations (taken in a
// second pass over the row, not from the mean of squares). Row r of the output is made from row
// rows[r] of x when `rows` is given. out may be x itself (float): every element is read by the
// thread that writes it, after the block has finished both sums.
template <typename TO, typename Acc>
__global__ void __launch_bounds__(256) layernorm_kernel(TO* __restrict__ out, const float* x, const float* __restrict__ w,
                                                        const float* __restrict__ b, const int32_t* __restrict__ rows,
                                                        int width, float eps, float out_scale) {
  __shared__ Acc scratch[4];
  const int r = blockIdx.x;
  const float* src = x + static_cast<int64_t>(rows ? rows[r] : r) * width;
  TO* dst = out + static_cast<int64_t>(r) * width;
  Acc s = 0;
  for (int c = threadIdx.x; c < width; c += 256) s += static_cast<Acc>(src[c]);
  const Acc mean = block_sum<Acc, 256>(s, scratch) / static_cast<Acc>(width);
  Acc ss = 0;
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc d = static_cast<Acc>(src[c]) - mean;
    ss += d * d;
  }
  const Acc var = block_sum<Acc, 256>(ss, scratch) / static_cast<Acc>(width);
  const Acc inv = static_cast<Acc>(1) / sqrt(var + static_cast<Acc>(eps));
  for (int c = threadIdx.x; c < width; c += 256) {
    const Acc y = (static_cast<Acc>(src[c]) - mean) * inv * static_cast<Acc>(w[c]) + static_cast<Acc>(b[c]);
    store_f32(dst + c, static_cast<float>(y * static_cast<Acc>(out_scale)));
  }
}

// ---- per-head unit norm, weight and gate -------------------------------------------------------
// out[t, h, :] = o[t, h, :] / sqrt(mean_j o[t, h, j]^2 + eps) * w[h, :] * silu(g[t, h, :]); w may be
// absent. One wavefront per (token, head). o is float (what a recurrence or attention left); g and
// out have the activation type.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) headnorm_gate_kernel(T* __restrict__ out, int64_t out_stride, const float* __restrict__ o,
                                                            const T* __restrict__ g, int64_t g_stride, const float* __restrict__ w,
                                                            int tokens, int heads, int dv, float eps, float out_scale, int parts, int64_t part_stride) {
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (unit >= static_cast<int64_t>(tokens) * heads) return;
  const int lane = threadIdx.x % kWave;
  const int t = static_cast<int>(unit / heads), h = static_cast<int>(unit % heads);
  const float* src = o + (static_cast<int64_t>(t) * heads + h) * dv;
  // (o may come in parts, left by blocks that each held a share of the key channels: they are added here, in their order)
  constexpr int kOwn = 4;      // values a lane keeps between the sum of squares and the scaling (heads up to 256 wide; wider ones are added again)
  float own[kOwn];
  Acc ss = 0;
#pragma unroll
  for (int c = 0; c < kOwn; ++c) {
    const int j = lane + c * kWave;
    float v = 0.f;
    if (j < dv)
      for (int p = 0; p < parts; ++p) v += src[p * part_stride + j];
    own[c] = v;
    ss += static_cast<Acc>(v) * static_cast<Acc>(v);
  }
  for (int j = lane + kOwn * kWave; j < dv; j += kWave) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += src[p * part_stride + j];
    ss += static_cast<Acc>(v) * static_cast<Acc>(v);
  }
  ss = wave_sum(ss);
  const Acc inv = static_cast<Acc>(1) / sqrt(ss / static_cast<Acc>(dv) + static_cast<Acc>(eps));
  const T* gate = g + static_cast<int64_t>(t) * g_stride + static_cast<int64_t>(h) * dv;
  T* dst = out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * dv;
  for (int j = lane; j < dv; j += kWave) {
    const Acc z = static_cast<Acc>(load_f32(gate + j));
    const Acc silu = z / (static_cast<Acc>(1) + exp(-z));
    float v = 0.f;
    if (j < kOwn * kWave) {
#pragma unroll
      for (int c = 0; c < kOwn; ++c)
        if (j == lane + c * kWave) v = own[c];
    } else {
      for (int p = 0; p < parts; ++p) v += src[p * part_stride + j];
    }
    Acc y = static_cast<Acc>(v) * inv;
    if (w) y *= static_cast<Acc>(w[h * dv + j]);
    store_f32(dst + j, static_cast<float>(y * silu * static_cast<Acc>(out_scale)));
  }
}

// ---- activations -------------------------------------------------------------------------------
// kind 0: xIELU with a = softplus(p) and b = 1/2 + softplus(q) given: z > 0: a z^2 + z/2; else b (exp(z) - 1 - z) + z/2.
// kind 1: tanh. In place or not; rows of `width` values with a row stride.
template <typename T, typename Acc>
__global__ void __launch_bounds__(256) activation_kernel(T* __restrict__ out, int64_t out_stride, const T* __restrict__ x, int64_t x_stride,
                                                         int64_t rows, int width, int kind, float a, float b) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (idx >= rows * width) return;
  const int64_t r = idx / width;
  const int c = static_cast<int>(idx % width);
  const Acc z = static_cast<Acc>(load_f32(x + r * x_stride + c));
  Acc y;
  if (kind == 0) {
    y = z > 0 ? static_cast<Acc>(a) * z * z + z / 2 : static_cast<Acc>(b) * (expm1(z) - z) + z / 2;
  } else {
    y = tanh(z);
  }
  store_f32(out + r * out_stride + c, static_cast<float>(y));
}

// ---- weighted average over depth -----------------------------------------------------------------
// stack[n - 1] = x; then x = sum_{j < n} w[j] * stack[j], j ascending. stack is [levels, elements].
// Without weights only the copy is made (the first level: what the layers start from).
template <typename Acc>
__global__ void __launch_bounds__(256) depth_average_kernel(float* __restrict__ x, float* __restrict__ stack, int64_t level_stride,
                                                            const float* __restrict__ w, int n, int64_t elements) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= elements) return;
  const float mine = x[e];
  stack[static_cast<int64_t>(n - 1) * level_stride + e] = mine;
  if (w == nullptr) return;
  Acc acc = 0;
  for (int j = 0; j < n - 1; ++j) acc += static_cast<Acc>(w[j]) * static_cast<Acc>(stack[static_cast<int64_t>(j) * level_stride + e]);
  acc += static_cast<Acc>(w[n - 1]) * static_cast<Acc>(mine);
  x[e] = static_cast<float>(acc);
}

// ---- residual += a * x + b * y; x *= s --------------------------------------------------------------
template <typename Acc>
__global__ void __launch_bounds__(256) add_scaled_kernel(float* __restrict__ residual, const float* __restrict__ x, float a,
                                                         const float* __restrict__ y, float b, int64_t elements) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= elements) return;
  Acc acc = static_cast<Acc>(a) * static_cast<Acc>(x[e]);
  if (y) acc += static_cast<Acc>(b) * static_cast<Acc>(y[e]);
  residual[e] = static_cast<float>(static_cast<Acc>(residual[e]) + acc);
}

__global__ void __launch_bounds__(256) scale_kernel(float* __restrict__ x, float s, int64_t elements) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e < elements) x[e] *= s;
}

}  // namespace alofa

using namespace alofa;

static inline unsigned blocks_of(int64_t n) { return static_cast<unsigned>((n + 255) / 256); }

extern "C" int alofa_layernorm(void* out, int out_dtype, const float* x, const float* w, const float* b, const int32_t* rows,
                               int n_rows, int width, float eps, float out_scale, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(n_rows >= 0 && width > 0 && eps > 0.f, "layernorm: bad sizes (rows=%d width=%d eps=%g)", n_rows, width, eps);
  ALOFA_REQUIRE(!exact || out_dtype == kF32, "layernorm: the exact path writes float32");
  if (n_rows == 0) return 0;
  if (exact) layernorm_kernel<float, double><<<n_rows, 256, 0, stream>>>(static_cast<float*>(out), x, w, b, rows, width, eps, out_scale);
  else if (out_dtype == kF32) layernorm_kernel<float, float><<<n_rows, 256, 0, stream>>>(static_cast<float*>(out), x, w, b, rows, width, eps, out_scale);
  else layernorm_kernel<bf16_t, float><<<n_rows, 256, 0, stream>>>(static_cast<bf16_t*>(out), x, w, b, rows, width, eps, out_scale);
  return check_launch("layernorm");
}

extern "C" int alofa_headnorm_gate(void* out, int64_t out_stride, const float* o, const void* g, int64_t g_stride, int dtype, const float* w,
                                   int tokens, int heads, int dv, float eps, float out_scale, int parts, int64_t part_stride, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(tokens >= 0 && heads > 0 && dv > 0 && eps > 0.f && parts >= 1, "headnorm_gate: bad sizes (tokens=%d heads=%d dv=%d)", tokens, heads, dv);
  ALOFA_REQUIRE(!exact || dtype == kF32, "headnorm_gate: the exact path is float32");
  if (tokens == 0) return 0;
  const unsigned grid = static_cast<unsigned>((static_cast<int64_t>(tokens) * heads + 3) / 4);
  if (exact) headnorm_gate_kernel<float, double><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, o, static_cast<const float*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride);
  else if (dtype == kF32) headnorm_gate_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, o, static_cast<const float*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride);
  else headnorm_gate_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, o, static_cast<const bf16_t*>(g), g_stride, w, tokens, heads, dv, eps, out_scale, parts, part_stride);
  return check_launch("headnorm_gate");
}

extern "C" int alofa_activation(void* out, int64_t out_stride, const void* x, int64_t x_stride, int dtype, int64_t rows, int width,
                                int kind, float a, float b, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(rows >= 0 && width > 0 && (kind == 0 || kind == 1), "activation: bad arguments (rows=%lld width=%d kind=%d)", (long long)rows, width, kind);
  ALOFA_REQUIRE(!exact || dtype == kF32, "activation: the exact path is float32");
  if (rows == 0) return 0;
  const unsigned grid = blocks_of(rows * width);
  if (exact) activation_kernel<float, double><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, static_cast<const float*>(x), x_stride, rows, width, kind, a, b);
  else if (dtype == kF32) activation_kernel<float, float><<<grid, 256, 0, stream>>>(static_cast<float*>(out), out_stride, static_cast<const float*>(x), x_stride, rows, width, kind, a, b);
  else activation_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(x), x_stride, rows, width, kind, a, b);
  return check_launch("activation");
}

extern "C" int alofa_depth_average(float* x, float* stack, int64_t level_stride, const float* w, int n, int64_t elements, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(n >= 1 && elements >= 0 && level_stride >= elements, "depth_average: bad sizes (n=%d elements=%lld stride=%lld)", n, (long long)elements, (long long)level_stride);
  if (elements == 0) return 0;
  if (exact) depth_average_kernel<double><<<blocks_of(elements), 256, 0, stream>>>(x, stack, level_stride, w, n, elements);
  else depth_average_kernel<float><<<blocks_of(elements), 256, 0, stream>>>(x, stack, level_stride, w, n, elements);
  return check_launch("depth_average");
}

extern "C" int alofa_add_scaled(float* residual, const float* x, float a, const float* y, float b, int64_t elements, int exact, hipStream_t stream) {
  ALOFA_REQUIRE(elements >= 0 && x != nullptr, "add_scaled: bad arguments");
  if (elements == 0) return 0;
  if (exact) add_scaled_kernel<double><<<blocks_of(elements), 256, 0, stream>>>(residual, x, a, y, b, elements);
  else add_scaled_kernel<float><<<blocks_of(elements), 256, 0, stream>>>(residual, x, a, y, b, elements);
  return check_launch("add_scaled");
}

extern "C" int alofa_scale(float* x, float s, int64_t elements, hipStream_t stream) {
  ALOFA_REQUIRE(elements >= 0, "scale: bad size");
  if (elements == 0) return 0;
  scale_kernel<<<blocks_of(elements), 256, 0, stream>>>(x, s, elements);
  return check_launch("scale");
}
