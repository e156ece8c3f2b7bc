// Attention without a softmax over the paged cache (see attention_sigmoid.h for what it
// computes): the write of keys and values into pages, and the plain kernel: one block per
// row does all heads, since the mixing of the heads' weights needs every head's weight of a
// key at once. It is the 32-bit path, the kernel of single rows, and takes the sizes the
// matrix-core kernel refuses.
//
// Keys are walked in tiles of 64 that start at the first visible position (the start of the
// row's chunk, or 0), so the order of every sum depends on the row's own position only, never
// on how a request was cut into steps or on what else is in the batch. Scores, weights and
// their mixing are 32-bit.
#include "attention_sigmoid.h"

namespace ninfer {

constexpr int kSigTile = 64;        // keys per tile
constexpr int kSigThreads = 256;
constexpr int kSigMaxOut = 16;      // outputs a thread may own: Hq * vdim <= 256 * 16

// k and v of every row into the request's pages.
template <typename T>
__global__ void sigmoid_kv_write_kernel(SigAttnArgs a) {
  const int t = blockIdx.x;
  const int pos = a.positions[t];
  const int page = a.block_table[(int64_t)a.row_seq[t] * a.bt_stride + pos / a.page_size];
  const int slot = pos % a.page_size;
  const T* row = (const T*)a.qkv + (int64_t)t * a.q_stride + a.Hq * a.dim;
  T* kp = (T*)a.kpool;
  T* vp = (T*)a.vpool;
  const int nk = a.Hkv * a.dim, nv = a.Hkv * a.vdim;
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int g = i / a.dim, d = i % a.dim;
    kp[(((int64_t)page * a.Hkv + g) * a.page_size + slot) * a.dim + d] = row[i];
  }
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const int g = i / a.vdim, d = i % a.vdim;
    vp[(((int64_t)page * a.Hkv + g) * a.page_size + slot) * a.vdim + d] = row[nk + i];
  }
}

template <typename T>
__global__ __launch_bounds__(kSigThreads) void sigmoid_attention_plain_kernel(SigAttnArgs a) {
  extern __shared__ float smem[];
  const int H = a.Hq, dim = a.dim, vdim = a.vdim;
  float* q_s = smem;                              // [H, dim]
  float* w_s = q_s + H * dim;                     // [H, 64] weights of the tile's keys
  float* m_s = w_s + H * kSigTile;                // [H, 64] mixed weights (unused without mix)
  float* mix_s = m_s + H * kSigTile;              // [H, H]
  int* slot_s = (int*)(mix_s + H * H);            // [64] page * page_size + slot of each key

  const int t = blockIdx.x, tid = threadIdx.x;
  const int per_kv = H / a.Hkv;
  const int pos = a.positions[t];
  const int first = a.chunk > 0 ? pos / a.chunk * a.chunk : 0;
  const int* bt = a.block_table + (int64_t)a.row_seq[t] * a.bt_stride;
  const T* kpool = (const T*)a.kpool;
  const T* vpool = (const T*)a.vpool;
  const T* qr = (const T*)a.qkv + (int64_t)t * a.q_stride;
  for (int e = tid; e < H * dim; e += kSigThreads) q_s[e] = to_f32(qr[e]);
  if (a.mix)
    for (int e = tid; e < H * H; e += kSigThreads) mix_s[e] = a.mix[e];
  const float* p_s = a.mix ? m_s : w_s;           // what the values are weighted by

  const int n_out = H * vdim;
  float acc[kSigMaxOut];
#pragma unroll
  for (int i = 0; i < kSigMaxOut; ++i) acc[i] = 0.f;

  for (int tile = first; tile <= pos; tile += kSigTile) {
    const int n_keys = min(kSigTile, pos - tile + 1);
    __syncthreads();   // the last tile's weights are read; (first tile) q_s and mix_s are written
    if (tid < kSigTile) {
      const int j = tile + tid;
      slot_s[tid] = tid < n_keys ? bt[j / a.page_size] * a.page_size + j % a.page_size : 0;
    }
    __syncthreads();
    // the weight of every (head, key) of the tile
    for (int e = tid; e < H * kSigTile; e += kSigThreads) {
      const int h = e / kSigTile, jj = e % kSigTile;
      float w = 0.f;
      if (jj < n_keys) {
        const int g = h / per_kv;
        const int page = slot_s[jj] / a.page_size, slot = slot_s[jj] % a.page_size;
        const T* kr = kpool + (((int64_t)page * a.Hkv + g) * a.page_size + slot) * dim;
        const float* qh = q_s + h * dim;
        float s = 0.f;
        for (int d = 0; d < dim; ++d) s = fmaf(qh[d], to_f32(kr[d]), s);
        s = s * a.scale + (a.head_bias ? a.head_bias[h] : 0.f);
        w = 1.f / (1.f + expf(-s));
      }
      w_s[e] = w;
    }
    __syncthreads();
    if (a.mix) {
      for (int e = tid; e < H * kSigTile; e += kSigThreads) {
        const int h = e / kSigTile, jj = e % kSigTile;
        float m = 0.f;
        for (int b = 0; b < H; ++b) m = fmaf(mix_s[h * H + b], w_s[b * kSigTile + jj], m);
        m_s[e] = m;
      }
      __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < kSigMaxOut; ++i) {
      const int e = tid + i * kSigThreads;
      if (e < n_out) {
        const int h = e / vdim, d = e % vdim, g = h / per_kv;
        const float* ph = p_s + h * kSigTile;
        float x = acc[i];
        for (int jj = 0; jj < n_keys; ++jj) {
          const int page = slot_s[jj] / a.page_size, slot = slot_s[jj] % a.page_size;
          const float v = to_f32(vpool[(((int64_t)page * a.Hkv + g) * a.page_size + slot) * vdim + d]);
          x = fmaf(ph[jj], v, x);
        }
        acc[i] = x;
      }
    }
  }
  T* orow = (T*)a.out + (int64_t)t * n_out;
#pragma unroll
  for (int i = 0; i < kSigMaxOut; ++i) {
    const int e = tid + i * kSigThreads;
    if (e < n_out) orow[e] = from_f32<T>(acc[i]);
  }
}

int sigmoid_attention_plain(const SigAttnArgs& a, hipStream_t stream) {
  const size_t lds = ((size_t)a.Hq * a.dim + 2 * a.Hq * kSigTile + a.Hq * a.Hq) * sizeof(float) +
                     kSigTile * sizeof(int);
  NINFER_REQUIRE(lds <= 64 * 1024 && a.Hq * a.vdim <= kSigThreads * kSigMaxOut,
                 "sigmoid_attention: %d heads of %d and %d numbers are more than the kernel holds",
                 a.Hq, a.dim, a.vdim);
  if (a.dtype == kF32)
    sigmoid_attention_plain_kernel<float><<<a.T, kSigThreads, lds, stream>>>(a);
  else
    sigmoid_attention_plain_kernel<bf16><<<a.T, kSigThreads, lds, stream>>>(a);
  NINFER_LAUNCH_CHECK();
  return 0;
}

static int sigmoid_check(const SigAttnArgs& a, const char* who) {
  NINFER_REQUIRE(a.T > 0 && a.S > 0 && a.Hq > 0 && a.Hkv > 0 && a.dim > 0 && a.vdim > 0 &&
                 a.page_size > 0, "%s: T=%d S=%d heads=%d/%d dim=%d vdim=%d page=%d must be positive",
                 who, a.T, a.S, a.Hq, a.Hkv, a.dim, a.vdim, a.page_size);
  NINFER_REQUIRE(a.Hq % a.Hkv == 0, "%s: %d heads are no multiple of %d kv heads", who, a.Hq, a.Hkv);
  NINFER_REQUIRE(a.dtype == kF32 || a.dtype == kBF16, "%s: unknown dtype %d", who, a.dtype);
  NINFER_REQUIRE(a.chunk >= 0, "%s: chunk %d is negative", who, a.chunk);
  NINFER_REQUIRE(a.q_stride >= a.Hq * a.dim, "%s: rows of %d numbers hold no %d x %d queries", who,
                 a.q_stride, a.Hq, a.dim);
  NINFER_REQUIRE(a.scale == a.scale, "%s: the scale is no number", who);
  return 0;
}

}  // namespace ninfer

using namespace ninfer;

extern "C" int ninfer_sigmoid_kv_write(const SigAttnArgs* a, hipStream_t stream) {
  int rc = sigmoid_check(*a, "sigmoid_kv_write");
  if (rc) return rc;
  NINFER_REQUIRE(a->q_stride >= (a->Hq + a->Hkv) * a->dim + a->Hkv * a->vdim,
                 "sigmoid_kv_write: rows of %d numbers hold no keys and values", a->q_stride);
  if (a->dtype == kF32) sigmoid_kv_write_kernel<float><<<a->T, 256, 0, stream>>>(*a);
  else sigmoid_kv_write_kernel<bf16><<<a->T, 256, 0, stream>>>(*a);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// 32-bit scratch the call needs (0: none): the partial outputs of the matrix-core kernel.
extern "C" long long ninfer_sigmoid_attention_workspace_floats(const SigAttnArgs* a) {
  if (sigmoid_check(*a, "sigmoid_attention")) return 0;
  if (a->force_plain || !sigmoid_attention_tiles_takes(*a)) return 0;
  const int n = sigmoid_attention_tiles_splits(*a);
  return n > 1 ? (long long)n * a->T * a->Hq * a->vdim : 0;
}

extern "C" int ninfer_sigmoid_attention(const SigAttnArgs* a, hipStream_t stream) {
  int rc = sigmoid_check(*a, "sigmoid_attention");
  if (rc) return rc;
  NINFER_REQUIRE(a->out && a->qkv && a->kpool && a->vpool, "sigmoid_attention: null tensors");
  if (!a->force_plain && sigmoid_attention_tiles_takes(*a)) {
    const int n = sigmoid_attention_tiles_splits(*a);
    if (n > 1)
      NINFER_REQUIRE(a->workspace && a->workspace_floats >= (int64_t)n * a->T * a->Hq * a->vdim,
                     "sigmoid_attention: the workspace is too small for %d parts", n);
    return sigmoid_attention_tiles(*a, a->workspace, n, stream);
  }
  return sigmoid_attention_plain(*a, stream);
}
