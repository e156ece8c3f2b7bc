// Row-wise kernels around a sublayer whose norm sits on its output:
//
//   short_conv     h_t + sum_j w[:, j] h_(t - taps + 1 + j): a causal convolution over the
//                  rows of each request, channel by channel, added to its input. The last
//                  taps - 1 inputs of a request are per-request state (32-bit), so a request
//                  may be cut into steps anywhere; before a request's start they are zero.
//   norm_add       x += y rsqrt(mean(y^2) + eps) g, g one number or one per channel; optionally
//                  with the row's mean taken off first (a layer norm), and with y a weighted
//                  sum of rows.
//   gated_rmsnorm  out = o rsqrt(mean(o^2) + eps) w sigmoid(g) (or w g sigmoid(g)), the norm
//                  over the whole row or over every group of columns (a head's) by itself.
//
// All sums are 32-bit and their order depends on the row alone (taps ascending; the block
// reduction's order depends on the width), never on how a request was cut or on the batch.
#include "common.h"

namespace ninfer {

// out[t, c] for all rows. Inputs before the step's first row of a request come from the
// request's state: state[slot][i * H + c] is the input at the request's position
// pos0 - (taps - 1) + i. With `update` (steps in which every request brings one row) the
// thread also shifts the state; otherwise short_conv_state_kernel does so afterwards.
template <typename T>
__global__ void short_conv_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                  float* __restrict__ state, int64_t state_stride,
                                  T* __restrict__ out, const int* __restrict__ row_seq,
                                  const int* __restrict__ seq_row_start,
                                  const int* __restrict__ seq_slots, int H, int taps, int update) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= H) return;
  const int s = row_seq[t];
  const int r0 = seq_row_start[s];
  const int i = t - r0;
  float* st = state + (int64_t)seq_slots[s] * state_stride;
  const float* wc = w + (int64_t)c * taps;
  const float cur = x[(int64_t)t * H + c];
  float acc = 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = i - (taps - 1 - j);
    const float v = src >= 0 ? x[(int64_t)(r0 + src) * H + c] : st[(int64_t)(taps - 1 + src) * H + c];
    acc = fmaf(wc[j], v, acc);
  }
  out[(int64_t)t * H + c] = from_f32<T>(cur + acc);
  if (update) {   // this row is the request's only one: the state moves on by one input
    for (int k = 0; k + 2 < taps; ++k) st[(int64_t)k * H + c] = st[(int64_t)(k + 1) * H + c];
    if (taps > 1) st[(int64_t)(taps - 2) * H + c] = cur;
  }
}

// state <- the last taps - 1 inputs of each request after this step's n rows. Entry k is the
// input at index n - (taps - 1) + k of the step's rows; a negative index is the old entry
// k + n, which lies above k, so ascending k never reads what it has written.
__global__ void short_conv_state_kernel(const float* __restrict__ x, float* __restrict__ state,
                                        int64_t state_stride,
                                        const int* __restrict__ seq_row_start,
                                        const int* __restrict__ seq_slots, int H, int taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= H) return;
  const int r0 = seq_row_start[s];
  const int n = seq_row_start[s + 1] - r0;
  float* st = state + (int64_t)seq_slots[s] * state_stride;
  for (int k = 0; k < taps - 1; ++k) {
    const int p = n - (taps - 1) + k;
    st[(int64_t)k * H + c] = p >= 0 ? x[(int64_t)(r0 + p) * H + c] : st[(int64_t)(k + n) * H + c];
  }
}

// x += norm(y) g with norm(y) = y rsqrt(mean(y^2) + eps), or with `center` the layer norm
// (y - mean) rsqrt(mean((y - mean)^2) + eps). y is a row of `y`, or with `w` the weighted sum of
// k rows, y_r = sum_j w[r, j] y[r k + j] (a sparse feed-forward's chosen experts), formed in
// 32-bit in the order of j. A thread keeps its (at most 8) numbers of the row in registers, in
// groups of VEC consecutive ones (VEC 4: whole 8- and 16-byte loads and stores).
constexpr int kNormAddPerThread = 8;
template <int VEC>
__device__ __forceinline__ void na_load(const float* p, float* f) {
  if constexpr (VEC == 4) {
    const float4 v = *(const float4*)p;
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
  } else {
    f[0] = p[0];
  }
}
template <int VEC>
__device__ __forceinline__ void na_load(const bf16* p, float* f) {
  if constexpr (VEC == 4) {
    const uint2 v = *(const uint2*)p;   // four bf16: the upper halves of four floats
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  } else {
    f[0] = to_f32(p[0]);
  }
}

template <typename T, int VEC>
__global__ void norm_add_kernel(float* __restrict__ x, const T* __restrict__ y,
                                const float* __restrict__ w, int k,
                                const float* __restrict__ gain, int gain_n, int H, float eps,
                                int center) {
  constexpr int G = kNormAddPerThread / VEC;
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  float vals[G][VEC];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < G; ++c) {
    const int i = VEC * (threadIdx.x + c * blockDim.x);
#pragma unroll
    for (int e = 0; e < VEC; ++e) vals[c][e] = 0.f;
    if (i < H) {
      if (w) {
        for (int j = 0; j < k; ++j) {
          float yv[VEC];
          na_load<VEC>(y + (r * k + j) * H + i, yv);
          const float wj = w[r * k + j];
#pragma unroll
          for (int e = 0; e < VEC; ++e) vals[c][e] = fmaf(wj, yv[e], vals[c][e]);
        }
      } else {
        na_load<VEC>(y + r * H + i, vals[c]);
      }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) sum += vals[c][e];
  }
  const float mean = center ? block_sum(sum, red) / (float)H : 0.f;
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < G; ++c) {
    const bool in = VEC * (threadIdx.x + c * blockDim.x) < H;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float d = in ? vals[c][e] - mean : 0.f;
      ss = fmaf(d, d, ss);
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)H + eps);
  float* xr = x + r * H;
#pragma unroll
  for (int c = 0; c < G; ++c) {
    const int i = VEC * (threadIdx.x + c * blockDim.x);
    if (i < H) {
      float xv[VEC], gv[VEC];
      na_load<VEC>(xr + i, xv);
      if (gain_n == 1) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) gv[e] = gain[0];
      } else {
        na_load<VEC>(gain + i, gv);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) xv[e] += (vals[c][e] - mean) * inv * gv[e];
      if constexpr (VEC == 4) *(float4*)(xr + i) = make_float4(xv[0], xv[1], xv[2], xv[3]);
      else xr[i] = xv[0];
    }
  }
}

template <typename T>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                     int gate_stride, const float* __restrict__ w,
                                     T* __restrict__ out, int N, float eps, int silu) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const float* orow = o + r * N;
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += blockDim.x) ss = fmaf(orow[i], orow[i], ss);
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)N + eps);
  const T* g = gate + r * gate_stride;
  for (int i = threadIdx.x; i < N; i += blockDim.x) {
    const float z = to_f32(g[i]);
    const float sg = (silu ? z : 1.f) / (1.f + expf(-z));
    out[r * N + i] = from_f32<T>(orow[i] * inv * w[i] * sg);
  }
}

// The same with the norm over every group of `group` neighbouring columns by itself (a head's
// values) and a weight of `group` numbers that all groups share: one wave per (row, group).
template <typename T>
__global__ __launch_bounds__(64) void gated_group_rmsnorm_kernel(
    const float* __restrict__ o, const T* __restrict__ gate, int gate_stride,
    const float* __restrict__ w, T* __restrict__ out, int N, int group, float eps, int silu) {
  const int64_t r = blockIdx.x;
  const int g0 = blockIdx.y * group, lane = threadIdx.x;
  const float* orow = o + r * N + g0;
  float ss = 0.f;
  for (int i = lane; i < group; i += 64) ss = fmaf(orow[i], orow[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.f / sqrtf(ss / (float)group + eps);
  const T* g = gate + r * gate_stride + g0;
  for (int i = lane; i < group; i += 64) {
    const float z = to_f32(g[i]);
    const float sg = (silu ? z : 1.f) / (1.f + expf(-z));
    out[r * N + g0 + i] = from_f32<T>(orow[i] * inv * w[i] * sg);
  }
}

static int row_block(int H) {
  int b = (H + 63) / 64 * 64;
  return b > 256 ? 256 : b;
}

}  // namespace ninfer

using namespace ninfer;

extern "C" int ninfer_short_conv(const float* x, const float* w, float* state,
                                 long long state_stride, void* out, const int* row_seq,
                                 const int* seq_row_start, const int* seq_slots, int T, int S,
                                 int H, int taps, int all_single, int dtype, hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && S > 0 && H > 0, "short_conv: T=%d S=%d H=%d must be positive", T, S, H);
  NINFER_REQUIRE(taps >= 1, "short_conv: %d taps", taps);
  NINFER_REQUIRE(state_stride >= (long long)(taps - 1) * H,
                 "short_conv: a request's state of %lld floats holds no %d x %d inputs",
                 state_stride, taps - 1, H);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "short_conv: unknown dtype %d", dtype);
  const int block = row_block(H);
  const dim3 grid(T, (H + block - 1) / block);
  if (dtype == kF32)
    short_conv_kernel<float><<<grid, block, 0, stream>>>(x, w, state, state_stride, (float*)out,
                                                         row_seq, seq_row_start, seq_slots, H,
                                                         taps, all_single);
  else
    short_conv_kernel<bf16><<<grid, block, 0, stream>>>(x, w, state, state_stride, (bf16*)out,
                                                        row_seq, seq_row_start, seq_slots, H, taps,
                                                        all_single);
  NINFER_LAUNCH_CHECK();
  if (!all_single && taps > 1) {
    short_conv_state_kernel<<<dim3(S, (H + block - 1) / block), block, 0, stream>>>(
        x, state, state_stride, seq_row_start, seq_slots, H, taps);
    NINFER_LAUNCH_CHECK();
  }
  return 0;
}

extern "C" int ninfer_norm_add(float* x, const void* y, const float* gain, int gain_n, int T, int H,
                               float eps, int dtype, int center, const float* w, int k,
                               hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && H > 0, "norm_add: T=%d H=%d must be positive", T, H);
  NINFER_REQUIRE(gain_n == 1 || gain_n == H, "norm_add: %d gains for %d channels", gain_n, H);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "norm_add: unknown dtype %d", dtype);
  NINFER_REQUIRE(H <= 1024 * kNormAddPerThread, "norm_add: width %d exceeds %d", H,
                 1024 * kNormAddPerThread);
  NINFER_REQUIRE(!w || k > 0, "norm_add: a weighted sum of %d rows", k);
  // groups of 4 consecutive numbers when every row stays 16-byte aligned
  auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  const bool vec = H % 4 == 0 && aligned(x) && aligned(y) && (gain_n == 1 || aligned(gain));
  const int per_thread = vec ? 4 : 1;
  int block = ((H + per_thread - 1) / per_thread + 63) / 64 * 64;
  if (block > 1024) block = 1024;
  NINFER_REQUIRE((int64_t)block * kNormAddPerThread >= H, "norm_add: width %d exceeds the kernel's", H);
  if (dtype == kF32) {
    if (vec) norm_add_kernel<float, 4><<<T, block, 0, stream>>>(x, (const float*)y, w, k, gain, gain_n, H, eps, center);
    else norm_add_kernel<float, 1><<<T, block, 0, stream>>>(x, (const float*)y, w, k, gain, gain_n, H, eps, center);
  } else {
    if (vec) norm_add_kernel<bf16, 4><<<T, block, 0, stream>>>(x, (const bf16*)y, w, k, gain, gain_n, H, eps, center);
    else norm_add_kernel<bf16, 1><<<T, block, 0, stream>>>(x, (const bf16*)y, w, k, gain, gain_n, H, eps, center);
  }
  NINFER_LAUNCH_CHECK();
  return 0;
}

// group 0 (or N): the norm over the whole row with a weight of N numbers; else over every
// group of `group` columns with a weight of `group` numbers. silu: the gate's factor is
// g sigmoid(g) instead of sigmoid(g).
extern "C" int ninfer_gated_rmsnorm(const float* o, const void* gate, int gate_stride,
                                    const float* w, void* out, int T, int N, float eps, int dtype,
                                    int group, int silu, hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && N > 0 && gate_stride >= N, "gated_rmsnorm: T=%d N=%d gate stride %d", T,
                 N, gate_stride);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "gated_rmsnorm: unknown dtype %d", dtype);
  NINFER_REQUIRE(group >= 0 && (group == 0 || N % group == 0),
                 "gated_rmsnorm: groups of %d columns do not fill rows of %d", group, N);
  if (group > 0 && group < N) {
    const dim3 grid(T, N / group);
    if (dtype == kF32)
      gated_group_rmsnorm_kernel<float><<<grid, 64, 0, stream>>>(o, (const float*)gate, gate_stride,
                                                                 w, (float*)out, N, group, eps, silu);
    else
      gated_group_rmsnorm_kernel<bf16><<<grid, 64, 0, stream>>>(o, (const bf16*)gate, gate_stride,
                                                                w, (bf16*)out, N, group, eps, silu);
    NINFER_LAUNCH_CHECK();
    return 0;
  }
  const int block = N >= 1024 ? 1024 : (N + 63) / 64 * 64;
  if (dtype == kF32)
    gated_rmsnorm_kernel<float><<<T, block, 0, stream>>>(o, (const float*)gate, gate_stride, w,
                                                         (float*)out, N, eps, silu);
  else
    gated_rmsnorm_kernel<bf16><<<T, block, 0, stream>>>(o, (const bf16*)gate, gate_stride, w,
                                                        (bf16*)out, N, eps, silu);
  NINFER_LAUNCH_CHECK();
  return 0;
}
