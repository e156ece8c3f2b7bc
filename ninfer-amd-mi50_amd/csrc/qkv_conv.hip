// What lies between the q/k/v projection and attention when the projected rows pass a short
// causal convolution over time first, in one kernel (a block per row, a wave per head):
//
//   y_t[c] = sum_j w[c, j] u_(t - taps + 1 + j)[c]        per channel c of the projected row u
//            (taps 0: y = u), zeros before a request's start; the taps - 1 projected rows
//            before a step's first row come from the request's state (32-bit), so a request may
//            be cut into steps anywhere;
//   query and key heads: y <- y rsqrt(mean(y^2) + eps) gain over the head's `dim` numbers (gains
//            null: no norm), then the first rot_dim numbers turn by pos * inv_freq[i]: pair i is
//            (i, i + rot_dim / 2), or the neighbours (2i, 2i + 1) when `interleaved`;
//   queries go to q_out [T, Hq * dim]; keys [dim] and values [vdim] (convolved only) go to the
//            request's pages of pools of their own. A layer that reads another layer's keys
//            and values brings rows of queries only (Hkv 0).
//
// A second kernel moves every request's state on to the step's last taps - 1 projected rows.
// All sums are 32-bit, in the order of the taps; the order never depends on how a request was
// cut or on the batch.
#include "common.h"

namespace ninfer {

struct QkvConvArgs {
  const void* u;            // [T, C] projected rows: Hq x dim, then Hkv x dim, then Hkv x vdim
  const float* w;           // [C, taps] or null
  float* state;             // [slots, state_stride]: (taps - 1) x C per request, or null
  int64_t state_stride;
  void* q_out;              // [T, Hq * dim]
  void* kpool;              // [pages, Hkv, page_size, dim]
  void* vpool;              // [pages, Hkv, page_size, vdim]
  const int* block_table;   // [S, bt_stride]
  const int* positions;     // [T]
  const int* row_seq;       // [T]
  const int* seq_row_start; // [S + 1]
  const int* seq_slots;     // [S]
  const float* q_gain;      // [dim] or null
  const float* k_gain;      // [dim] or null
  const float* inv_freq;    // [rot_dim / 2] or null
  int bt_stride;
  int T;
  int S;
  int Hq;
  int Hkv;                  // 0: the rows hold queries only
  int dim;
  int vdim;
  int taps;
  int rot_dim;
  int interleaved;
  int page_size;
  int dtype;
  float eps;
  int all_single;           // every request of the step brings one row
};

constexpr int kConvPerLane = 8;   // heads of up to 512 numbers
constexpr int kConvWaves = 4;

// A block per row: cosine and sine of the row's angles once for all heads, then wave w takes
// heads w, w + 4, ... With `update` (steps in which every request brings one row) the lane
// that convolves a channel also moves the channel's state on; otherwise qkv_conv_state_kernel
// does so afterwards.
template <typename T>
__global__ __launch_bounds__(64 * kConvWaves) void qkv_conv_kernel(QkvConvArgs a, int maxd, int update) {
  extern __shared__ float smem[];
  float* trig = smem;                                   // [rot_dim]: cos, then sin
  float* head_s = smem + a.rot_dim + (threadIdx.x >> 6) * maxd;   // [maxd] of this wave
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int C = a.Hq * a.dim + a.Hkv * (a.dim + a.vdim);
  const int total = a.Hq + 2 * a.Hkv;
  const int s = a.row_seq[t];
  const int r0 = a.seq_row_start[s];
  const int i_row = t - r0;
  const int pos = a.positions[t];
  const int half = a.rot_dim / 2;
  const T* u = (const T*)a.u;
  float* st = a.state ? a.state + (int64_t)a.seq_slots[s] * a.state_stride : nullptr;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float sn, cs;
    sincosf((float)pos * a.inv_freq[i], &sn, &cs);
    trig[i] = cs;
    trig[half + i] = sn;
  }
  int page = 0, slot = 0;
  if (a.Hkv > 0) {
    page = a.block_table[(int64_t)s * a.bt_stride + pos / a.page_size];
    slot = pos % a.page_size;
  }
  for (int hd0 = 0; hd0 < total; hd0 += kConvWaves) {
    const int hd = hd0 + wave;
    const bool live = hd < total;
    // which head: a query's, a key's or a value's
    int kind = 2, col0 = 0, n = 0;
    if (live) {
      if (hd < a.Hq) { kind = 0; col0 = hd * a.dim; n = a.dim; }
      else if (hd < a.Hq + a.Hkv) { kind = 1; col0 = hd * a.dim; n = a.dim; }
      else { col0 = (a.Hq + a.Hkv) * a.dim + (hd - a.Hq - a.Hkv) * a.vdim; n = a.vdim; }
    }
    float vals[kConvPerLane];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kConvPerLane; ++i) {
      const int d = lane + 64 * i;
      float y = 0.f;
      if (d < n) {
        const int ch = col0 + d;
        if (a.taps > 0) {
          const float* wc = a.w + (int64_t)ch * a.taps;
          for (int j = 0; j < a.taps; ++j) {
            const int src = i_row - (a.taps - 1 - j);
            const float v = src >= 0 ? to_f32(u[(int64_t)(r0 + src) * C + ch])
                                     : st[(int64_t)(a.taps - 1 + src) * C + ch];
            y = fmaf(wc[j], v, y);
          }
          if (update && a.taps > 1) {   // this row is the request's only one: the state moves on by one row
            for (int k = 0; k + 2 < a.taps; ++k) st[(int64_t)k * C + ch] = st[(int64_t)(k + 1) * C + ch];
            st[(int64_t)(a.taps - 2) * C + ch] = to_f32(u[(int64_t)t * C + ch]);
          }
        } else {
          y = to_f32(u[(int64_t)t * C + ch]);
        }
      }
      vals[i] = y;
      ss = fmaf(y, y, ss);
    }
    const float* gain = kind == 0 ? a.q_gain : kind == 1 ? a.k_gain : nullptr;
    if (gain) {
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / (float)n + a.eps);
#pragma unroll
      for (int i = 0; i < kConvPerLane; ++i) {
        const int d = lane + 64 * i;
        if (d < n) vals[i] *= inv * gain[d];
      }
    }
    T* dst = nullptr;
    if (live) {
      const int g = kind == 1 ? hd - a.Hq : hd - a.Hq - a.Hkv;
      dst = kind == 0 ? (T*)a.q_out + (int64_t)t * a.Hq * a.dim + col0
          : kind == 1 ? (T*)a.kpool + (((int64_t)page * a.Hkv + g) * a.page_size + slot) * a.dim
                      : (T*)a.vpool + (((int64_t)page * a.Hkv + g) * a.page_size + slot) * a.vdim;
    }
    const int rot = kind == 2 ? 0 : a.rot_dim;
#pragma unroll
    for (int i = 0; i < kConvPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < rot) head_s[d] = vals[i];
    }
    __syncthreads();   // (the first time round it also publishes trig)
#pragma unroll
    for (int i = 0; i < kConvPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < rot) {
        int p;
        bool first;
        float x, y;
        if (a.interleaved) { p = d >> 1; first = !(d & 1); x = head_s[2 * p]; y = head_s[2 * p + 1]; }
        else { p = d < half ? d : d - half; first = d < half; x = head_s[p]; y = head_s[p + half]; }
        const float cs = trig[p], sn = trig[half + p];
        vals[i] = first ? x * cs - y * sn : y * cs + x * sn;
      }
    }
    __syncthreads();   // the heads' numbers are read: the next head may overwrite them
#pragma unroll
    for (int i = 0; i < kConvPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < n) dst[d] = from_f32<T>(vals[i]);
    }
  }
}

// state <- the last taps - 1 projected rows of each request after this step's n rows. Entry k is
// the row at index n - (taps - 1) + k of the step's rows; a negative index is the old entry
// k + n, which lies above k, so ascending k never reads what it has written.
template <typename T>
__global__ void qkv_conv_state_kernel(QkvConvArgs a, int C) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int r0 = a.seq_row_start[s];
  const int n = a.seq_row_start[s + 1] - r0;
  const T* u = (const T*)a.u;
  float* st = a.state + (int64_t)a.seq_slots[s] * a.state_stride;
  for (int k = 0; k < a.taps - 1; ++k) {
    const int p = n - (a.taps - 1) + k;
    st[(int64_t)k * C + c] = p >= 0 ? to_f32(u[(int64_t)(r0 + p) * C + c]) : st[(int64_t)(k + n) * C + c];
  }
}

}  // namespace ninfer

using namespace ninfer;

extern "C" int ninfer_qkv_conv(const QkvConvArgs* args, hipStream_t stream) {
  const QkvConvArgs& a = *args;
  NINFER_REQUIRE(a.T > 0 && a.S > 0 && a.Hq > 0 && a.Hkv >= 0 && a.dim > 0 && a.vdim > 0,
                 "qkv_conv: T=%d S=%d heads=%d/%d dim=%d vdim=%d", a.T, a.S, a.Hq, a.Hkv, a.dim, a.vdim);
  NINFER_REQUIRE(a.dim <= 64 * kConvPerLane && a.vdim <= 64 * kConvPerLane,
                 "qkv_conv: heads of %d and %d numbers exceed %d", a.dim, a.vdim, 64 * kConvPerLane);
  NINFER_REQUIRE(a.taps >= 0 && (a.taps == 0 || a.w), "qkv_conv: %d taps without weights", a.taps);
  const int C = a.Hq * a.dim + a.Hkv * (a.dim + a.vdim);
  NINFER_REQUIRE(a.taps <= 1 || (a.state && a.state_stride >= (int64_t)(a.taps - 1) * C),
                 "qkv_conv: a request's state holds no %d x %d projected numbers", a.taps - 1, C);
  NINFER_REQUIRE(a.rot_dim >= 0 && a.rot_dim % 2 == 0 && a.rot_dim <= a.dim &&
                 (a.rot_dim == 0 || a.inv_freq), "qkv_conv: %d turning numbers of %d", a.rot_dim, a.dim);
  NINFER_REQUIRE((a.q_gain == nullptr) == (a.k_gain == nullptr) || a.Hkv == 0,
                 "qkv_conv: both heads' norms or neither");
  NINFER_REQUIRE(a.Hkv == 0 || (a.kpool && a.vpool && a.block_table && a.page_size > 0),
                 "qkv_conv: keys and values without pages");
  NINFER_REQUIRE(a.dtype == kF32 || a.dtype == kBF16, "qkv_conv: unknown dtype %d", a.dtype);
  const int maxd = a.dim > a.vdim ? a.dim : a.vdim;
  const size_t lds = (size_t)(a.rot_dim + kConvWaves * maxd) * sizeof(float);
  NINFER_REQUIRE(a.all_single == 0 || a.all_single == 1, "qkv_conv: all_single is a flag");
  const int update = a.all_single;
  if (a.dtype == kF32) qkv_conv_kernel<float><<<a.T, 64 * kConvWaves, lds, stream>>>(a, maxd, update);
  else qkv_conv_kernel<bf16><<<a.T, 64 * kConvWaves, lds, stream>>>(a, maxd, update);
  NINFER_LAUNCH_CHECK();
  if (a.taps > 1 && !update) {
    const dim3 sgrid(a.S, (C + 255) / 256);
    if (a.dtype == kF32) qkv_conv_state_kernel<float><<<sgrid, 256, 0, stream>>>(a, C);
    else qkv_conv_state_kernel<bf16><<<sgrid, 256, 0, stream>>>(a, C);
    NINFER_LAUNCH_CHECK();
  }
  return 0;
}
