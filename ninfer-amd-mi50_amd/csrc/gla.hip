// Gated linear attention: linear attention whose state decays per key channel by a factor
// that every token brings, token by token:
//
//   alpha_t = sigmoid(z_t)^(1 / tau)                     (per head and key channel, in (0, 1))
//   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T              (S: [dim, vdim] per head, 32-bit)
//   o_t = S_t^T (q_t q_scale)
//
// z comes in 32-bit (the decay's logits after their bias); the decay is formed here as
// exp(log_sigmoid(z) / tau). The state comes from and returns to the request's slot, so a
// request may be cut into steps anywhere and every row sees exactly the sums it would see in
// one piece.
//
// A block of four waves owns 64 value columns of one (request, head) and walks the request's
// rows of the step in order; a wave owns 16 of the columns. Lane (part, col) keeps S[d][col]
// for the DPL key channels d = part DPL .. in registers, updates them and forms its part of
// o_t[col]; the four parts are added by two lane exchanges. q, k and the decay of a row are
// staged in LDS by the block's threads, a channel each (two buffers, one barrier a row); the
// rows come from global memory eight at a time, one batch ahead of the one being computed, so
// that the loads' latency is paid once per batch. The order of every sum depends on dim alone.
#include "common.h"

namespace ninfer {

constexpr int kGlaCols = 16;    // value columns per wave
constexpr int kGlaParts = 4;    // parts of the key channels, one per 16 lanes
constexpr int kGlaWaves = 4;    // waves per block
constexpr int kGlaBatch = 8;    // rows fetched at a time

__device__ __forceinline__ float log_sigmoid(float z) {
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

struct GlaArgs {
  const void* qkv;        // [T, stride] rows: q at q_off, k at k_off (H x dim), v at v_off (H x vdim)
  const float* z;         // [T, H * dim] the decay's logits
  float* state;           // + slot * state_stride: [H, dim, vdim]
  float* out;             // [T, H * vdim]
  const int* seq_row_start;
  const int* seq_slots;
  int64_t state_stride;
  int stride, q_off, k_off, v_off;
  int H, dim, vdim;
  float inv_tau, q_scale;
};

template <typename T, int DPL>
__global__ __launch_bounds__(64 * kGlaWaves) void gla_seq_kernel(GlaArgs a) {
  constexpr int DIM = DPL * kGlaParts;            // channels held (>= dim; the rest stay 0)
  static_assert(DIM <= 64 * kGlaWaves, "a thread stages one channel");
  __shared__ __attribute__((aligned(16))) float q_s[2][DIM], k_s[2][DIM], a_s[2][DIM];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = (blockIdx.z * kGlaWaves + wave) * kGlaCols + (lane & (kGlaCols - 1));
  const int part = lane / kGlaCols;
  const bool has_col = col < a.vdim;
  const int r0 = a.seq_row_start[s], n = a.seq_row_start[s + 1] - r0;
  const int dim = a.dim, vdim = a.vdim;
  float* st = a.state + (int64_t)a.seq_slots[s] * a.state_stride + (int64_t)h * dim * vdim;

  float S[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = part * DPL + i;
    S[i] = has_col && d < dim ? st[(int64_t)d * vdim + col] : 0.f;
  }
  // the batch of rows a thread fetches ahead: q, k and the decay's logit of its channel (thread
  // tid looks after channel tid), and v of its column
  const bool stages = tid < DIM, in_dim = tid < dim;
  float fq[kGlaBatch], fk[kGlaBatch], fz[kGlaBatch], fv[kGlaBatch];
  auto fetch = [&](int first) {
#pragma unroll
    for (int j = 0; j < kGlaBatch; ++j) {
      const int row = r0 + min(first + j, n - 1);   // (rows beyond the last are fetched again, not used)
      const T* r = (const T*)a.qkv + (int64_t)row * a.stride;
      fq[j] = in_dim ? to_f32(r[a.q_off + h * dim + tid]) : 0.f;
      fk[j] = in_dim ? to_f32(r[a.k_off + h * dim + tid]) : 0.f;
      fz[j] = in_dim ? a.z[((int64_t)row * a.H + h) * dim + tid] : 0.f;
      fv[j] = has_col ? to_f32(r[a.v_off + h * vdim + col]) : 0.f;
    }
  };
  if (n > 0) fetch(0);
  for (int base = 0; base < n; base += kGlaBatch) {
    float cq[kGlaBatch], ck[kGlaBatch], ca[kGlaBatch], cv[kGlaBatch];
#pragma unroll
    for (int j = 0; j < kGlaBatch; ++j) {
      cq[j] = fq[j] * a.q_scale;
      ck[j] = fk[j];
      ca[j] = in_dim ? expf(log_sigmoid(fz[j]) * a.inv_tau) : 1.f;
      cv[j] = fv[j];
    }
    if (base + kGlaBatch < n) fetch(base + kGlaBatch);
#pragma unroll
    for (int j = 0; j < kGlaBatch; ++j) {
      if (base + j >= n) break;
      const int b = j & 1;
      if (stages) {
        q_s[b][tid] = cq[j];
        k_s[b][tid] = ck[j];
        a_s[b][tid] = ca[j];
      }
      // (a barrier that waits for LDS traffic only: the batch on its way and the outputs' stores
      // stay in flight)
      lds_barrier();   // the row is in LDS; the other buffer's readers are done
      const float v_t = cv[j];
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const int d = part * DPL + i;
        const float sn = fmaf(a_s[b][d], S[i], k_s[b][d] * v_t);
        S[i] = sn;
        o = fmaf(sn, q_s[b][d], o);
      }
      o += __shfl_xor(o, 16, 64);
      o += __shfl_xor(o, 32, 64);
      if (part == 0 && has_col) a.out[((int64_t)(r0 + base + j) * a.H + h) * vdim + col] = o;
    }
  }
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = part * DPL + i;
    if (has_col && d < dim) st[(int64_t)d * vdim + col] = S[i];
  }
}

}  // namespace ninfer

using namespace ninfer;

// qkv: [T, stride] rows of the activation dtype with the heads' q at column q_off, k at k_off
// (heads x dim each) and v at v_off (heads x vdim); z: [T, heads * dim] 32-bit; out:
// [T, heads * vdim] 32-bit.
extern "C" int ninfer_gated_linear_attention(const void* qkv, int stride, int q_off, int k_off,
                                             int v_off, const float* z, float tau, float q_scale,
                                             float* state, long long state_stride, float* out,
                                             const int* seq_row_start, const int* seq_slots,
                                             int T, int S, int H, int dim, int vdim, int dtype,
                                             hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && S > 0 && H > 0 && dim > 0 && vdim > 0,
                 "gated_linear_attention: T=%d S=%d heads=%d dim=%d vdim=%d must be positive", T,
                 S, H, dim, vdim);
  NINFER_REQUIRE(dim <= 256, "gated_linear_attention: %d key channels exceed 256", dim);
  NINFER_REQUIRE(tau > 0.f, "gated_linear_attention: tau (%g) must be positive", tau);
  NINFER_REQUIRE(state_stride >= (long long)H * dim * vdim,
                 "gated_linear_attention: a request's state of %lld floats holds no %d x %d x %d",
                 state_stride, H, dim, vdim);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "gated_linear_attention: unknown dtype %d", dtype);
  GlaArgs a;
  a.qkv = qkv, a.z = z, a.state = state, a.out = out;
  a.seq_row_start = seq_row_start, a.seq_slots = seq_slots, a.state_stride = state_stride;
  a.stride = stride, a.q_off = q_off, a.k_off = k_off, a.v_off = v_off;
  a.H = H, a.dim = dim, a.vdim = vdim, a.inv_tau = 1.f / tau, a.q_scale = q_scale;
  const int cols = kGlaCols * kGlaWaves;
  const dim3 grid(S, H, (vdim + cols - 1) / cols);
#define NINFER_GLA(DPL)                                                             \
  do {                                                                              \
    if (dtype == kF32) gla_seq_kernel<float, DPL><<<grid, 64 * kGlaWaves, 0, stream>>>(a);      \
    else gla_seq_kernel<bf16, DPL><<<grid, 64 * kGlaWaves, 0, stream>>>(a);                     \
  } while (0)
  if (dim <= 16) NINFER_GLA(4);
  else if (dim <= 32) NINFER_GLA(8);
  else if (dim <= 64) NINFER_GLA(16);
  else if (dim <= 128) NINFER_GLA(32);
  else NINFER_GLA(64);
#undef NINFER_GLA
  NINFER_LAUNCH_CHECK();
  return 0;
}
