// Routed feed-forward ("mixture of experts"): the router with its selection rule, the experts'
// products for the (token, taken expert) pairs of a step, and the weighted sum.
//
// Router, all in 32-bit: z = R x, s = sigmoid(z).  The experts form `groups` equal groups of
// neighbours; a group's mark is the sum of its two largest s (its one s if it has one member);
// only experts of the `keep` groups with the largest marks can be taken; the `top` of them with
// the largest s are, with weights s / (sum of the taken s + 1e-20) * route_scale.  Equal values go
// to the lower index.  groups == 1 is plain top-k.
#include "common.hpp"

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 32

template <typename T>
__device__ __forceinline__ float lanes_dot(const T* __restrict__ a, const T* __restrict__ b, int n, int lane) {
  float s = 0.f;
  for (int k = lane; k < n; k += TS_WAVE) s = fmaf(to_float(a[k]), to_float(b[k]), s);
  return wave_sum(s);
}

// Index of the largest of the values the lanes hold (value, index pairs; index < 2^24), the
// lower index among equals; every lane returns it.  A lane without a candidate passes -inf.
__device__ __forceinline__ int wave_argmax(float value, int index, float& best) {
  best = wave_max(value);
  const float mine = (value == best) ? -(float)index : -16777216.f;
  return (int)(-wave_max(mine));
}

// One block of 256 threads per token.
template <typename T>
__global__ void __launch_bounds__(256)
moe_route_kernel(int* __restrict__ taken, float* __restrict__ weights, float* __restrict__ extra_gate,
                 const T* __restrict__ x, const T* __restrict__ router, const T* __restrict__ extra, int width,
                 int experts, int top, int groups, int keep, float route_scale) {
  __shared__ float score[MOE_MAX_EXPERTS];
  __shared__ float mark[MOE_MAX_EXPERTS];   // per group
  __shared__ int open_group[MOE_MAX_EXPERTS];
  const int t = blockIdx.x;
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x % TS_WAVE, waves = blockDim.x / TS_WAVE;
  const T* row = x + (size_t)t * width;
  for (int e = wave; e < experts; e += waves) {
    const float z = lanes_dot(router + (size_t)e * width, row, width, lane);
    if (lane == 0) score[e] = 1.f / (1.f + expf(-z));
  }
  if (extra_gate && wave == waves - 1) {
    const float z = lanes_dot(extra, row, width, lane);
    if (lane == 0) extra_gate[t] = 1.f / (1.f + expf(-z));
  }
  __syncthreads();
  // The selection is the first wavefront's; the others only keep the barriers company.
  const bool lead = wave == 0;
  const int size = experts / groups;
  if (lead) {
    for (int g = lane; g < groups; g += TS_WAVE) {
      float a = -INFINITY, b = -INFINITY;  // largest, second
      for (int i = 0; i < size; ++i) {
        const float s = score[g * size + i];
        if (s > a) { b = a; a = s; } else if (s > b) { b = s; }
      }
      mark[g] = size > 1 ? a + b : a;
      open_group[g] = keep >= groups ? 1 : 0;
    }
  }
  __syncthreads();
  if (keep < groups) {
    for (int round = 0; round < keep; ++round) {
      if (lead) {
        float mine = -INFINITY;
        int at = 0;
        for (int g = lane; g < groups; g += TS_WAVE)
          if (!open_group[g] && mark[g] > mine) { mine = mark[g]; at = g; }
        float best;
        const int g = wave_argmax(mine, at, best);
        if (lane == 0) open_group[g] = 1;
      }
      __syncthreads();
    }
  }
  float total = 0.f;
  float kept_score = 0.f;  // lane r holds the score of the r-th taken expert
  int kept_index = 0;
  for (int round = 0; round < top; ++round) {
    if (lead) {
      float mine = -INFINITY;
      int at = 0;
      for (int e = lane; e < experts; e += TS_WAVE)
        if (open_group[e / size] && score[e] > mine) { mine = score[e]; at = e; }
      float best;
      const int e = wave_argmax(mine, at, best);
      if (lane == round) { kept_score = best; kept_index = e; }
      total += best;
      if (lane == 0) score[e] = -INFINITY;  // taken
    }
    __syncthreads();
  }
  if (lead && lane < top) {
    taken[(size_t)t * top + lane] = kept_index;
    weights[(size_t)t * top + lane] = kept_score / (total + 1e-20f) * route_scale;
  }
}

extern "C" int ts_moe_route(int* taken, float* weights, float* extra_gate, const void* x, const void* router,
                            const void* extra, int tokens, int width, int experts, int top, int groups, int keep,
                            float route_scale, int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!taken || !weights || !x || !router || (extra_gate && !extra)) return TS_ERR_ARG;
  if (experts < 1 || experts > MOE_MAX_EXPERTS || top < 1 || top > MOE_MAX_TOP || groups < 1 || experts % groups != 0 ||
      keep < 1 || keep > groups || top > (experts / groups) * keep || width < 1)
    return TS_ERR_SHAPE;
  if (dtype == TS_F32)
    hipLaunchKernelGGL(moe_route_kernel<float>, dim3(tokens), dim3(256), 0, stream, taken, weights, extra_gate, (const float*)x, (const float*)router, (const float*)extra, width, experts, top, groups, keep, route_scale);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream, taken, weights, extra_gate, (const bf16_t*)x, (const bf16_t*)router, (const bf16_t*)extra, width, experts, top, groups, keep, route_scale);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// The experts' products pair by pair: pair p = (token p / top, its (p % top)-th taken expert e).
// Weights are stacked over the experts, [E, N, K].  out[p, n] = W[e][n] . in[row(p)] with row(p) =
// p / in_share (the token's activations for the first product: in_share = top; the pair's own row
// for the second: in_share = 1).  GATED: N = 2 I rows alternate gate, up and the output is
// gated_unit(gate, up) of the run type, [P, I]; else the output is 32-bit, [P, N].  A block
// stages the input row in LDS as 32-bit and its wavefronts walk the rows of a slice of N: the
// weights stream once per pair, which is what a step of few tokens costs anyway.
// ---------------------------------------------------------------------------------------------
#define MOE_ROWS_PER_BLOCK 32

template <typename T>
__device__ __forceinline__ float row_dot_staged(const T* __restrict__ w, const float* __restrict__ xs, int k, int lane);

template <>
__device__ __forceinline__ float row_dot_staged<float>(const float* __restrict__ w, const float* __restrict__ xs, int k,
                                                       int lane) {
  float s = 0.f;
  for (int i = lane; i < k; i += TS_WAVE) s = fmaf(w[i], xs[i], s);
  return wave_sum(s);
}

template <>
__device__ __forceinline__ float row_dot_staged<bf16_t>(const bf16_t* __restrict__ w, const float* __restrict__ xs, int k,
                                                        int lane) {
  float s = 0.f;
  if ((k & 7) == 0 && ((uintptr_t)w & 15) == 0) {
    for (int i = lane * 8; i < k; i += TS_WAVE * 8) {
      const ts_u32x4 v = load_once16(w + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s = fmaf(__uint_as_float(v[e] << 16), xs[i + 2 * e], s);
        s = fmaf(__uint_as_float(v[e] & 0xffff0000u), xs[i + 2 * e + 1], s);
      }
    }
  } else {
    for (int i = lane; i < k; i += TS_WAVE) s = fmaf(to_float(w[i]), xs[i], s);
  }
  return wave_sum(s);
}

template <typename T, bool GATED>
__global__ void __launch_bounds__(256)
moe_pair_rows_kernel(void* __restrict__ out_any, const T* __restrict__ in, const T* __restrict__ weight,
                     const int* __restrict__ taken, int in_share, int n, int k, int experts, GluRule rule) {
  extern __shared__ float xs[];
  const int pair = blockIdx.x;
  const int e = taken[pair];
  const T* row = in + (size_t)(pair / in_share) * k;
  for (int i = threadIdx.x; i < k; i += blockDim.x) xs[i] = to_float(row[i]);
  __syncthreads();
  if (e < 0 || e >= experts) return;  // a host error; nothing is read out of bounds
  const int wave = threadIdx.x / TS_WAVE, lane = threadIdx.x % TS_WAVE, waves = blockDim.x / TS_WAVE;
  const T* w = weight + (size_t)e * n * k;
  if (GATED) {
    const int units = n / 2;
    T* out = (T*)out_any + (size_t)pair * units;
    const int first = blockIdx.y * MOE_ROWS_PER_BLOCK;
    for (int i = first + wave; i < min(first + MOE_ROWS_PER_BLOCK, units); i += waves) {
      const float g = row_dot_staged<T>(w + (size_t)(2 * i) * k, xs, k, lane);
      const float u = row_dot_staged<T>(w + (size_t)(2 * i + 1) * k, xs, k, lane);
      if (lane == 0) out[i] = from_float<T>(gated_unit(g, u, rule));
    }
  } else {
    float* out = (float*)out_any + (size_t)pair * n;
    const int first = blockIdx.y * MOE_ROWS_PER_BLOCK;
    for (int i = first + wave; i < min(first + MOE_ROWS_PER_BLOCK, n); i += waves) {
      const float y = row_dot_staged<T>(w + (size_t)i * k, xs, k, lane);
      if (lane == 0) out[i] = y;
    }
  }
}

extern "C" int ts_moe_pair_rows(void* out, const void* in, const void* weight, const int* taken, int pairs,
                                int in_share, int n, int k, int experts, int gated, float steepness, float limit,
                                float up_shift, int dtype, hipStream_t stream) {
  if (pairs == 0) return TS_OK;
  if (!out || !in || !weight || !taken) return TS_ERR_ARG;
  if (n < 1 || k < 1 || k > 12288 || in_share < 1 || experts < 1 || (gated && (n & 1))) return TS_ERR_SHAPE;
  const GluRule rule = {steepness, limit, up_shift};
  const int outputs = gated ? n / 2 : n;
  const dim3 grid(pairs, (outputs + MOE_ROWS_PER_BLOCK - 1) / MOE_ROWS_PER_BLOCK), block(256);
  if (grid.y > 65535) return TS_ERR_SHAPE;
  const size_t lds = (size_t)k * sizeof(float);
  if (dtype == TS_F32 && gated)
    hipLaunchKernelGGL((moe_pair_rows_kernel<float, true>), grid, block, lds, stream, out, (const float*)in, (const float*)weight, taken, in_share, n, k, experts, rule);
  else if (dtype == TS_F32)
    hipLaunchKernelGGL((moe_pair_rows_kernel<float, false>), grid, block, lds, stream, out, (const float*)in, (const float*)weight, taken, in_share, n, k, experts, rule);
  else if (dtype == TS_BF16 && gated)
    hipLaunchKernelGGL((moe_pair_rows_kernel<bf16_t, true>), grid, block, lds, stream, out, (const bf16_t*)in, (const bf16_t*)weight, taken, in_share, n, k, experts, rule);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL((moe_pair_rows_kernel<bf16_t, false>), grid, block, lds, stream, out, (const bf16_t*)in, (const bf16_t*)weight, taken, in_share, n, k, experts, rule);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}

// ---------------------------------------------------------------------------------------------
// out[t, :] = sum_j weights[t, j] * pair_out[t * top + j, :]  (+ extra_gate[t] * extra[t, :]),
// 32-bit, summed in the order j = 0, 1, ..; `extra` (the shared expert's output) is of type P: T,
// or `splits` 32-bit partial sums `split_stride` elements apart.
// ---------------------------------------------------------------------------------------------
template <typename P>
__global__ void moe_combine_kernel(float* __restrict__ out, const float* __restrict__ pair_out,
                                   const float* __restrict__ weights, const P* __restrict__ extra, int splits,
                                   size_t split_stride, const float* __restrict__ extra_gate, int top, int width) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float s = 0.f;
    for (int j = 0; j < top; ++j)
      s = fmaf(weights[(size_t)t * top + j], pair_out[((size_t)t * top + j) * width + i], s);
    if (extra) {
      float x = 0.f;
      for (int sp = 0; sp < splits; ++sp) x += to_float(extra[(size_t)sp * split_stride + (size_t)t * width + i]);
      s = fmaf(extra_gate ? extra_gate[t] : 1.f, x, s);
    }
    out[(size_t)t * width + i] = s;
  }
}

extern "C" int ts_moe_combine(float* out, const float* pair_out, const float* weights, const void* extra,
                              int extra_f32, int splits, long split_stride, const float* extra_gate, int tokens,
                              int top, int width, int dtype, hipStream_t stream) {
  if (tokens == 0) return TS_OK;
  if (!out || !pair_out || !weights || top < 1 || width < 1 || splits < 1) return TS_ERR_ARG;
  const dim3 grid(tokens), block(256);
  if (!extra || extra_f32 || dtype == TS_F32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, grid, block, 0, stream, out, pair_out, weights, (const float*)extra, splits, (size_t)split_stride, extra_gate, top, width);
  else if (dtype == TS_BF16)
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, grid, block, 0, stream, out, pair_out, weights, (const bf16_t*)extra, splits, (size_t)split_stride, extra_gate, top, width);
  else
    return TS_ERR_DTYPE;
  return ts_launch_status();
}
