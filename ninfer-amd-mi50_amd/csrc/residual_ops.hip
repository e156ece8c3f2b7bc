// Row-wise kernels around the 32-bit residual stream that models of parallel sublayers use:
// the embedding with a scale and a hashed table of token pairs, two streams laid side by
// side as the input of a product, the sum of both sublayers' results with a scale per
// column, a tanh cap in place, and the square of relu in place.
#include "common.h"

namespace ninfer {

// x[t,:] = table[token[t],:] * scale + pair_table[row(t),:], in 32-bit.
// row(t) = (prev * mul_prev + token * mul_cur) mod buckets with prev the token before t in
// its request: the row above when t is not the first row of its request in this step, else
// what the request's state holds (previous token + 1 as an integer; 0: the request starts
// here, and the row is `buckets`, the table's last). pair_table null: no such term.
template <typename T>
__global__ void embed_pairs_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                                   float* __restrict__ out, int H, float scale,
                                   const T* __restrict__ pair_table, int buckets, int mul_prev,
                                   int mul_cur, const int* __restrict__ row_seq,
                                   const int* __restrict__ seq_row_start,
                                   const int* __restrict__ seq_slots, const int* __restrict__ state,
                                   int64_t state_stride) {
  const int64_t t = blockIdx.x;
  const int tok = tokens[t];
  const T* src = table + (int64_t)tok * H;
  float* dst = out + t * H;
  if (!pair_table) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = to_f32(src[i]) * scale;
    return;
  }
  const int s = row_seq[t];
  int prev;   // previous token + 1
  if (t > seq_row_start[s]) prev = tokens[t - 1] + 1;
  else prev = state[(int64_t)seq_slots[s] * state_stride];
  int64_t row = buckets;
  if (prev > 0)
    row = (int64_t)(((uint64_t)(prev - 1) * (uint64_t)mul_prev + (uint64_t)tok * (uint64_t)mul_cur) %
                    (uint64_t)buckets);
  const T* psrc = pair_table + row * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    dst[i] = to_f32(src[i]) * scale + to_f32(psrc[i]);
}

// After the rows are embedded: every request's state takes its last token of the step (+ 1).
__global__ void embed_pairs_state_kernel(const int* __restrict__ tokens,
                                         const int* __restrict__ seq_row_start,
                                         const int* __restrict__ seq_slots, int* __restrict__ state,
                                         int64_t state_stride, int S) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= S) return;
  state[(int64_t)seq_slots[s] * state_stride] = tokens[seq_row_start[s + 1] - 1] + 1;
}

// out[t, :H] = a[t, :], out[t, H:] = b[t, :]: two 32-bit streams side by side in the
// activation dtype, the input of one product over both.
template <typename T>
__global__ void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                   T* __restrict__ out, int H) {
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    out[t * 2 * H + i] = from_f32<T>(a[t * H + i]);
    out[t * 2 * H + H + i] = from_f32<T>(b[t * H + i]);
  }
}

// residual[t,c] += s1[c] * a[t,c] + s2[c] * f(t,c), in 32-bit, where f is dense rows
// (`dense`), or the weighted sum of a sparse feed-forward's rows
// sum_j w[t,j] * y[t*k + j, c] + sigmoid(gate[t * gate_stride]) * shared[t,c], or nothing.
// s1 / s2 null: factor 1.
template <typename T>
__global__ void scaled_sum_add_kernel(float* __restrict__ residual, const T* __restrict__ a,
                                      const float* __restrict__ s1, const T* __restrict__ dense,
                                      const T* __restrict__ y, const float* __restrict__ w, int k,
                                      const T* __restrict__ shared, const float* __restrict__ gate,
                                      int gate_stride, const float* __restrict__ s2, int H) {
  const int64_t t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= H) return;
  float m = a ? to_f32(a[t * H + i]) * (s1 ? s1[i] : 1.f) : 0.f;
  float f = 0.f;
  bool has_f = false;
  if (dense) {
    f = to_f32(dense[t * H + i]);
    has_f = true;
  } else if (y) {
    for (int j = 0; j < k; ++j) f += w[t * k + j] * to_f32(y[(t * k + j) * H + i]);
    if (shared) {
      const float g = gate ? 1.f / (1.f + expf(-gate[t * gate_stride])) : 1.f;
      f += g * to_f32(shared[t * H + i]);
    }
    has_f = true;
  }
  if (has_f) m += f * (s2 ? s2[i] : 1.f);
  residual[t * H + i] += m;
}

// What the gated sum adds: residual[t,c] += mult (c1(t,c) a[t,c] + c2(t,c) f(t,c)) in 32-bit,
// with c = sigmoid(g[t,c] + b[c]) from a gate's logits g (rows of the activation dtype) and
// bias b, or 1 without a gate; f is dense rows, or the weighted sum of a sparse
// feed-forward's rows sum_j w[t,j] y[t k + j, c], where a choice j with ids[t,j] >= real
// stands for an expert that hands its input back: its term is w[t,j] xin[t,c].
struct GatedSumArgs {
  float* residual;
  const void* a;        // [T, H] or null
  const void* g1;       // [T, H] logits of a's gate, or null
  const float* b1;      // [H] or null
  const void* dense;    // [T, H] or null
  const void* y;        // [T k, H] or null
  const float* w;       // [T, k]
  const int* ids;       // [T, k] or null (every choice has a row of y)
  const void* xin;      // [T, H] what the experts read (with ids)
  const void* g2;       // [T, H] logits of f's gate, or null
  const float* b2;      // [H] or null
  int T, H, k, real, dtype;
  float mult;
};

template <typename T>
__global__ void gated_sum_add_kernel(GatedSumArgs p) {
  const int64_t t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  const int H = p.H;
  if (i >= H) return;
  float m = 0.f;
  if (p.a) {
    m = to_f32(((const T*)p.a)[t * H + i]);
    if (p.g1) m *= 1.f / (1.f + expf(-(to_f32(((const T*)p.g1)[t * H + i]) + (p.b1 ? p.b1[i] : 0.f))));
  }
  float f = 0.f;
  bool has_f = false;
  if (p.dense) {
    f = to_f32(((const T*)p.dense)[t * H + i]);
    has_f = true;
  } else if (p.y) {
    const T* y = (const T*)p.y;
    for (int j = 0; j < p.k; ++j) {
      const bool back = p.ids && p.ids[t * p.k + j] >= p.real;
      const float v = back ? to_f32(((const T*)p.xin)[t * H + i]) : to_f32(y[(t * p.k + j) * H + i]);
      f = fmaf(p.w[t * p.k + j], v, f);
    }
    has_f = true;
  }
  if (has_f) {
    if (p.g2) f *= 1.f / (1.f + expf(-(to_f32(((const T*)p.g2)[t * H + i]) + (p.b2 ? p.b2[i] : 0.f))));
    m += f;
  }
  p.residual[t * H + i] += p.mult * m;
}

// x <- cap * tanh(x / cap), in place (32-bit numbers).
__global__ void tanh_cap_kernel(float* __restrict__ x, int64_t n, float cap) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

// x <- max(x, 0)^2, in place.
template <typename T>
__global__ void relu_square_kernel(T* __restrict__ x, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const float v = fmaxf(to_f32(x[i]), 0.f);
    x[i] = from_f32<T>(v * v);
  }
}

}  // namespace ninfer

using namespace ninfer;

// state: one 32-bit integer per slot at state + slot * state_stride (in integers); null with
// pair_table null.
extern "C" int ninfer_embed_pairs(const int* tokens, const void* table, float* out, int T, int H,
                                  int dtype, float scale, const void* pair_table, int buckets,
                                  int mul_prev, int mul_cur, const int* row_seq,
                                  const int* seq_row_start, const int* seq_slots, int S, int* state,
                                  long long state_stride, hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && H > 0, "embed_pairs: T=%d H=%d must be positive", T, H);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "embed_pairs: unknown dtype %d", dtype);
  NINFER_REQUIRE(!pair_table || (buckets > 0 && mul_prev >= 0 && mul_cur >= 0 && row_seq &&
                                 seq_row_start && seq_slots && state && S > 0),
                 "embed_pairs: a table of pairs needs its buckets (%d), multipliers, the step's "
                 "requests and their state", buckets);
  if (dtype == kF32)
    embed_pairs_kernel<float><<<T, 256, 0, stream>>>(
        tokens, (const float*)table, out, H, scale, (const float*)pair_table, buckets, mul_prev,
        mul_cur, row_seq, seq_row_start, seq_slots, state, state_stride);
  else
    embed_pairs_kernel<bf16><<<T, 256, 0, stream>>>(
        tokens, (const bf16*)table, out, H, scale, (const bf16*)pair_table, buckets, mul_prev,
        mul_cur, row_seq, seq_row_start, seq_slots, state, state_stride);
  NINFER_LAUNCH_CHECK();
  if (pair_table) {
    embed_pairs_state_kernel<<<(S + 63) / 64, 64, 0, stream>>>(tokens, seq_row_start, seq_slots,
                                                               state, state_stride, S);
    NINFER_LAUNCH_CHECK();
  }
  return 0;
}

extern "C" int ninfer_concat_rows(const float* a, const float* b, void* out, int T, int H, int dtype,
                                  hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && H > 0, "concat_rows: T=%d H=%d must be positive", T, H);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "concat_rows: unknown dtype %d", dtype);
  if (dtype == kF32) concat_rows_kernel<float><<<T, 256, 0, stream>>>(a, b, (float*)out, H);
  else concat_rows_kernel<bf16><<<T, 256, 0, stream>>>(a, b, (bf16*)out, H);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_scaled_sum_add(float* residual, const void* a, const float* s1,
                                     const void* dense, const void* y, const float* w, int k,
                                     const void* shared, const float* gate, int gate_stride,
                                     const float* s2, int T, int H, int dtype, hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && H > 0, "scaled_sum_add: T=%d H=%d must be positive", T, H);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "scaled_sum_add: unknown dtype %d", dtype);
  NINFER_REQUIRE(!(dense && y), "scaled_sum_add: dense rows or a weighted sum, not both");
  NINFER_REQUIRE(!y || (w && k > 0), "scaled_sum_add: a weighted sum needs weights and k=%d > 0", k);
  dim3 grid(T, (H + 255) / 256);
  if (dtype == kF32)
    scaled_sum_add_kernel<float><<<grid, 256, 0, stream>>>(
        residual, (const float*)a, s1, (const float*)dense, (const float*)y, w, k,
        (const float*)shared, gate, gate_stride, s2, H);
  else
    scaled_sum_add_kernel<bf16><<<grid, 256, 0, stream>>>(
        residual, (const bf16*)a, s1, (const bf16*)dense, (const bf16*)y, w, k,
        (const bf16*)shared, gate, gate_stride, s2, H);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_gated_sum_add(const GatedSumArgs* p, hipStream_t stream) {
  NINFER_REQUIRE(p->T > 0 && p->H > 0, "gated_sum_add: T=%d H=%d must be positive", p->T, p->H);
  NINFER_REQUIRE(p->dtype == kF32 || p->dtype == kBF16, "gated_sum_add: unknown dtype %d", p->dtype);
  NINFER_REQUIRE(!(p->dense && p->y), "gated_sum_add: dense rows or a weighted sum, not both");
  NINFER_REQUIRE(!p->y || (p->w && p->k > 0), "gated_sum_add: a weighted sum needs weights and k=%d > 0", p->k);
  NINFER_REQUIRE(!p->ids || (p->xin && p->real >= 0), "gated_sum_add: experts that hand their input "
                 "back need that input");
  NINFER_REQUIRE(p->mult == p->mult, "gated_sum_add: the multiplier is no number");
  dim3 grid(p->T, (p->H + 255) / 256);
  if (p->dtype == kF32) gated_sum_add_kernel<float><<<grid, 256, 0, stream>>>(*p);
  else gated_sum_add_kernel<bf16><<<grid, 256, 0, stream>>>(*p);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_tanh_cap(float* x, long long n, float cap, hipStream_t stream) {
  NINFER_REQUIRE(n > 0 && cap > 0.f, "tanh_cap: n=%lld and the cap (%g) must be positive", n, cap);
  tanh_cap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, n, cap);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_relu_square(void* x, long long n, int dtype, hipStream_t stream) {
  NINFER_REQUIRE(n > 0, "relu_square: n=%lld must be positive", n);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "relu_square: unknown dtype %d", dtype);
  if (dtype == kF32) relu_square_kernel<float><<<(unsigned)((n + 255) / 256), 256, 0, stream>>>((float*)x, n);
  else relu_square_kernel<bf16><<<(unsigned)((n + 255) / 256), 256, 0, stream>>>((bf16*)x, n);
  NINFER_LAUNCH_CHECK();
  return 0;
}
