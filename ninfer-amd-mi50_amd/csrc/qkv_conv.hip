// What lies between the q/k/v projection and attention when the projected rows pass a short
// causal convolution over time first, in one kernel (a wave per row and head):
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
  const float* wt;          // the same transposed, [taps, C], or null (the kernel of whole pieces reads it)
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
  int force_plain;          // tests: 1 the kernel of a wave per head, 2 the kernel of whole pieces
                            // whatever the row count (where it takes the sizes)
};

constexpr int kConvPerLane = 8;   // heads of up to 512 numbers
constexpr int kConvWaves = 4;

// A block per row and four heads (a wave each): cosine and sine of the row's angles once for
// the block's heads. With `update` (steps in which every request brings one row) the lane
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
  {
    const int hd = blockIdx.y * kConvWaves + wave;
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
    __syncthreads();   // (it also publishes trig)
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
#pragma unroll
    for (int i = 0; i < kConvPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < n) dst[d] = from_f32<T>(vals[i]);
    }
  }
}

// The same for bfloat16 rows whose heads are multiples of 8 numbers: a block per row, a thread
// per piece of 8 consecutive channels (one 16-byte load per tap, one 16-byte store), the row's
// convolved numbers in LDS in 32-bit between the two phases: convolution and sums of squares,
// then norm, rotation (partners and angles from LDS) and the stores.
constexpr int kConvRowThreads = 256;
typedef unsigned int conv_u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void conv_unpack(conv_u32x4 v, float* f) {
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

__global__ __launch_bounds__(kConvRowThreads) void qkv_conv_rows_kernel(QkvConvArgs a, int update) {
  extern __shared__ float smem[];
  const int C = a.Hq * a.dim + a.Hkv * (a.dim + a.vdim);
  const int pieces = C / 8;
  float* row_s = smem;                 // [C] the convolved row
  float* ss_s = row_s + C;             // [pieces] sums of squares
  float* trig = ss_s + pieces;         // [rot_dim]: cos, then sin
  const int t = blockIdx.x, tid = threadIdx.x;
  const int s = a.row_seq[t];
  const int r0 = a.seq_row_start[s];
  const int i_row = t - r0;
  const int pos = a.positions[t];
  const int half = a.rot_dim / 2;
  const unsigned short* u = (const unsigned short*)a.u;
  float* st = a.state ? a.state + (int64_t)a.seq_slots[s] * a.state_stride : nullptr;
  for (int i = tid; i < half; i += kConvRowThreads) {
    float sn, cs;
    sincosf((float)pos * a.inv_freq[i], &sn, &cs);
    trig[i] = cs;
    trig[half + i] = sn;
  }
  for (int p = tid; p < pieces; p += kConvRowThreads) {
    const int ch = 8 * p;
    float y[8];
    if (a.taps > 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = 0.f;
      for (int j = 0; j < a.taps; ++j) {
        const int src = i_row - (a.taps - 1 - j);
        float v[8];
        if (src >= 0) {
          conv_unpack(*(const conv_u32x4*)(u + (int64_t)(r0 + src) * C + ch), v);
        } else {
          const float* sr = st + (int64_t)(a.taps - 1 + src) * C + ch;
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = sr[e];
        }
        const float4 w0 = *(const float4*)(a.wt + (int64_t)j * C + ch);
        const float4 w1 = *(const float4*)(a.wt + (int64_t)j * C + ch + 4);
        y[0] = fmaf(w0.x, v[0], y[0]); y[1] = fmaf(w0.y, v[1], y[1]);
        y[2] = fmaf(w0.z, v[2], y[2]); y[3] = fmaf(w0.w, v[3], y[3]);
        y[4] = fmaf(w1.x, v[4], y[4]); y[5] = fmaf(w1.y, v[5], y[5]);
        y[6] = fmaf(w1.z, v[6], y[6]); y[7] = fmaf(w1.w, v[7], y[7]);
      }
      if (update && a.taps > 1) {   // this row is the request's only one: the state moves on by one row
        float cur[8];
        conv_unpack(*(const conv_u32x4*)(u + (int64_t)t * C + ch), cur);
        for (int k = 0; k + 2 < a.taps; ++k)
#pragma unroll
          for (int e = 0; e < 8; ++e) st[(int64_t)k * C + ch + e] = st[(int64_t)(k + 1) * C + ch + e];
#pragma unroll
        for (int e = 0; e < 8; ++e) st[(int64_t)(a.taps - 2) * C + ch + e] = cur[e];
      }
    } else {
      conv_unpack(*(const conv_u32x4*)(u + (int64_t)t * C + ch), y);
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(y[e], y[e], ss);
    *(float4*)(row_s + ch) = make_float4(y[0], y[1], y[2], y[3]);
    *(float4*)(row_s + ch + 4) = make_float4(y[4], y[5], y[6], y[7]);
    ss_s[p] = ss;
  }
  __syncthreads();
  int page = 0, slot = 0;
  if (a.Hkv > 0) {
    page = a.block_table[(int64_t)s * a.bt_stride + pos / a.page_size];
    slot = pos % a.page_size;
  }
  const int nq = a.Hq * a.dim, nk = a.Hkv * a.dim;
  for (int p = tid; p < pieces; p += kConvRowThreads) {
    const int ch = 8 * p;
    // which head, and where in it
    int kind, hd, d0, n;
    if (ch < nq) { kind = 0; hd = ch / a.dim; d0 = ch - hd * a.dim; n = a.dim; }
    else if (ch < nq + nk) { kind = 1; hd = (ch - nq) / a.dim; d0 = ch - nq - hd * a.dim; n = a.dim; }
    else { kind = 2; hd = (ch - nq - nk) / a.vdim; d0 = ch - nq - nk - hd * a.vdim; n = a.vdim; }
    const float* head = row_s + ch - d0;
    const float* gain = kind == 0 ? a.q_gain : kind == 1 ? a.k_gain : nullptr;
    float inv = 1.f;
    if (gain) {
      float ss = 0.f;
      const float* hs = ss_s + (ch - d0) / 8;
      for (int i = 0; i < n / 8; ++i) ss += hs[i];   // the same order in every thread of the head
      inv = 1.f / sqrtf(ss / (float)n + a.eps);
    }
    const int rot = kind == 2 ? 0 : a.rot_dim;
    union { __bf16 b[8]; conv_u32x4 v; } out;
    // the piece's own numbers, normed; a piece lies wholly inside or outside the turning part
    // and its partners (d + half, d - half, or its own neighbours) are one piece too, since
    // rot_dim / 2 is a multiple of 8 or the pairs are neighbours
    float x[8], gn[8];
    {
      const float4 h0 = *(const float4*)(head + d0), h1 = *(const float4*)(head + d0 + 4);
      x[0] = h0.x; x[1] = h0.y; x[2] = h0.z; x[3] = h0.w; x[4] = h1.x; x[5] = h1.y; x[6] = h1.z; x[7] = h1.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) gn[e] = 1.f;
      if (gain) {
        const float4 g0 = *(const float4*)(gain + d0), g1 = *(const float4*)(gain + d0 + 4);
        gn[0] = g0.x; gn[1] = g0.y; gn[2] = g0.z; gn[3] = g0.w; gn[4] = g1.x; gn[5] = g1.y; gn[6] = g1.z; gn[7] = g1.w;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] *= inv * gn[e];
    }
    if (d0 < rot) {
      if (a.interleaved) {
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const float cs = trig[(d0 + e) >> 1], sn = trig[half + ((d0 + e) >> 1)];
          const float u0 = x[e], u1 = x[e + 1];
          x[e] = u0 * cs - u1 * sn;
          x[e + 1] = u1 * cs + u0 * sn;
        }
      } else {
        const bool first = d0 < half;
        const int o0 = first ? d0 + half : d0 - half;
        const float4 h0 = *(const float4*)(head + o0), h1 = *(const float4*)(head + o0 + 4);
        float y[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
        if (gain) {
          const float4 g0 = *(const float4*)(gain + o0), g1 = *(const float4*)(gain + o0 + 4);
          y[0] *= g0.x; y[1] *= g0.y; y[2] *= g0.z; y[3] *= g0.w; y[4] *= g1.x; y[5] *= g1.y; y[6] *= g1.z; y[7] *= g1.w;
        }
        const int p0 = first ? d0 : d0 - half;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float cs = trig[p0 + e], sn = trig[half + p0 + e];
          x[e] = first ? x[e] * cs - y[e] * inv * sn : x[e] * cs + y[e] * inv * sn;
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) out.b[e] = (__bf16)x[e];
    unsigned short* dst =
        kind == 0 ? (unsigned short*)a.q_out + (int64_t)t * nq + ch
        : kind == 1 ? (unsigned short*)a.kpool + (((int64_t)page * a.Hkv + hd) * a.page_size + slot) * a.dim + d0
                    : (unsigned short*)a.vpool + (((int64_t)page * a.Hkv + hd) * a.page_size + slot) * a.vdim + d0;
    *(conv_u32x4*)dst = out.v;
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
  const size_t row_lds = (size_t)(C + C / 8 + a.rot_dim) * sizeof(float);
  // whole pieces of 8: heads, and the turning part's halves unless the pairs are neighbours
  const bool pieces = a.dim % 8 == 0 && a.vdim % 8 == 0 && a.rot_dim % (a.interleaved ? 8 : 16) == 0 &&
                      (a.taps == 0 || a.wt);
  // (few rows: a block per row is too few blocks, and each walks its pieces in two rounds of
  // dependent loads; a wave per row and head then finishes sooner: 8 to 10 against 14 to 16 us
  // at 8 and 64 rows of 24 heads, but 48 against 16 us at 2,048 rows)
  if (a.dtype == kBF16 && pieces && row_lds <= 64 * 1024 && (a.T >= 256 || a.force_plain == 2) && a.force_plain != 1) {
    qkv_conv_rows_kernel<<<a.T, kConvRowThreads, row_lds, stream>>>(a, update);
    NINFER_LAUNCH_CHECK();
  } else {
  const dim3 grid(a.T, (a.Hq + 2 * a.Hkv + kConvWaves - 1) / kConvWaves);
  if (a.dtype == kF32) qkv_conv_kernel<float><<<grid, 64 * kConvWaves, lds, stream>>>(a, maxd, update);
  else qkv_conv_kernel<bf16><<<grid, 64 * kConvWaves, lds, stream>>>(a, maxd, update);
  NINFER_LAUNCH_CHECK();
  }
  if (a.taps > 1 && !update) {
    const dim3 sgrid(a.S, (C + 255) / 256);
    if (a.dtype == kF32) qkv_conv_state_kernel<float><<<sgrid, 256, 0, stream>>>(a, C);
    else qkv_conv_state_kernel<bf16><<<sgrid, 256, 0, stream>>>(a, C);
    NINFER_LAUNCH_CHECK();
  }
  return 0;
}
