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

// ---- prompt portions in chunks of 16 rows, on the 32-bit matrix instruction ---------------------
//
// With b_i = sum of ln alpha over the rows 0 .. i of a chunk (per key channel, <= 0) and the
// state S before the chunk, the recurrence written out is
//
//   o_i = (q_i * e^(b_i))^T S  +  sum_{j <= i} A[i][j] v_j,   A[i][j] = sum_d q_i[d] k_j[d] e^(b_i[d] - b_j[d])
//   S' = diag(e^(b_(L-1))) S + sum_j (k_j * e^(b_(L-1) - b_j)) v_j^T
//
// Every exponent is <= 0, so nothing grows, however strong the decay. A first kernel, one block
// per (chunk, head) and so as wide as the step, forms q e^b, k e^(b_last - b), e^b and A in
// 32-bit: A not from exponentials but as the recurrence does, by multiplying k_j with the decays
// of the rows that follow it, one after the other. A second kernel walks a request's chunks
// in order: a wave keeps 16 value columns of the state in the accumulators of
// v_mfma_f32_16x16x4_f32 (they are that instruction's second operand as they are: the order of
// a sum's terms is free), and a chunk costs it dim / 4 + 4 products for the outputs and
// dim / 4 for the state, with the operands of the next chunk on their way meanwhile. Nothing
// is rounded to a shorter type.
namespace ninfer {

typedef float gla_f32x4 __attribute__((ext_vector_type(4)));
constexpr int kGlaChunk = 16;
constexpr int kGlaChunkMaxDim = 128;

struct GlaChunkArgs {
  GlaArgs g;
  float* qe;     // [H, T, dim]  q q_scale e^b  (a chunk of a head is one piece of memory)
  float* ke;     // [H, T, dim]  k e^(b_last - b)
  float* eb;     // [H, T, dim]  e^b
  float* A;      // [H, T, 16]
  int T, S;
};

// The request and the first row of chunk `c` of the step (chunks are counted request after
// request); false if the step has fewer chunks.
__device__ __forceinline__ bool gla_find_chunk(const int* seq_row_start, int S, int c, int* r0,
                                               int* i0, int* n) {
  for (int s = 0; s < S; ++s) {
    const int a = seq_row_start[s], len = seq_row_start[s + 1] - a;
    const int chunks = (len + kGlaChunk - 1) / kGlaChunk;
    if (c < chunks) {
      *r0 = a, *i0 = c * kGlaChunk, *n = len;
      return true;
    }
    c -= chunks;
  }
  return false;
}

template <typename T>
__global__ __launch_bounds__(256) void gla_chunk_prepare_kernel(GlaChunkArgs a) {
  __shared__ float q_s[kGlaChunk][kGlaChunkMaxDim], k_s[kGlaChunk][kGlaChunkMaxDim];
  __shared__ float al_s[kGlaChunk][kGlaChunkMaxDim], b_s[kGlaChunk][kGlaChunkMaxDim];
  int r0, i0, n;
  if (!gla_find_chunk(a.g.seq_row_start, a.S, blockIdx.x, &r0, &i0, &n)) return;
  const int h = blockIdx.y, tid = threadIdx.x;
  const int dim = a.g.dim, H = a.g.H;
  const int L = min(kGlaChunk, n - i0), base = r0 + i0;
  // 1. the rows' q, k and decays; rows beyond the chunk's last count as absent (k = 0, alpha = 1)
  for (int e = tid; e < kGlaChunk * dim; e += 256) {
    const int t = e / dim, d = e % dim;
    float qv = 0.f, kv = 0.f, g = 0.f;
    if (t < L) {
      const T* r = (const T*)a.g.qkv + (int64_t)(base + t) * a.g.stride;
      qv = to_f32(r[a.g.q_off + h * dim + d]) * a.g.q_scale;
      kv = to_f32(r[a.g.k_off + h * dim + d]);
      g = log_sigmoid(a.g.z[((int64_t)(base + t) * H + h) * dim + d]) * a.g.inv_tau;
    }
    q_s[t][d] = qv, k_s[t][d] = kv, al_s[t][d] = expf(g), b_s[t][d] = g;
  }
  __syncthreads();
  // 2. b: the running sum of the logarithms, a channel per thread
  if (tid < dim) {
    float b = 0.f;
#pragma unroll
    for (int t = 0; t < kGlaChunk; ++t) {
      b += b_s[t][tid];
      b_s[t][tid] = b;
    }
  }
  __syncthreads();
  // 3. the scaled rows
  for (int e = tid; e < L * dim; e += 256) {
    const int t = e / dim, d = e % dim;
    const float eb = expf(b_s[t][d]);
    const int64_t at = ((int64_t)h * a.T + base + t) * dim + d;
    a.qe[at] = q_s[t][d] * eb;
    a.ke[at] = k_s[t][d] * expf(b_s[L - 1][d] - b_s[t][d]);
    a.eb[at] = eb;
  }
  // 4. A: thread (j, part) carries k_j times the decays since row j for the channels part,
  // part + 16, ..; the sixteen parts of a (row, j) are added by lane exchanges
  {
    const int j = tid >> 4, part = tid & 15;
    constexpr int PER = kGlaChunkMaxDim / 16;
    float kp[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int d = part + 16 * i;
      kp[i] = d < dim ? k_s[j][d] : 0.f;
    }
    for (int t = 0; t < L; ++t) {
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int d = part + 16 * i;
        if (d < dim) {
          if (t > j) kp[i] *= al_s[t][d];
          acc = fmaf(q_s[t][d], kp[i], acc);
        }
      }
      acc += __shfl_xor(acc, 1, 64);
      acc += __shfl_xor(acc, 2, 64);
      acc += __shfl_xor(acc, 4, 64);
      acc += __shfl_xor(acc, 8, 64);
      if (part == 0) a.A[((int64_t)h * a.T + base + t) * kGlaChunk + j] = j <= t ? acc : 0.f;
    }
  }
}

// A chunk's operands as the lanes of a wave hold them. Lane (c, g) = (lane % 16, lane / 16).
template <int DT>
struct GlaChunkRegs {
  gla_f32x4 q[DT];    // qe[row c][16 dt + 4 g ..]
  gla_f32x4 e[DT];    // eb[last row][16 dt + 4 g ..]
  float k[4][DT];     // ke[row 4 g + x][16 dt + c]
  gla_f32x4 A;        // A[row c][4 g ..]
  float v[4];         // v[row 4 g + x][column c of the wave]
};

template <typename T, int DT>
__global__ __launch_bounds__(64 * kGlaWaves) void gla_chunk_scan_kernel(GlaChunkArgs a) {
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int col = (blockIdx.z * kGlaWaves + wave) * kGlaCols + c;
  const int dim = a.g.dim, vdim = a.g.vdim, H = a.g.H;
  const bool has_col = col < vdim;
  const int r0 = a.g.seq_row_start[s], n = a.g.seq_row_start[s + 1] - r0;
  float* st = a.g.state + (int64_t)a.g.seq_slots[s] * a.g.state_stride + (int64_t)h * dim * vdim;
  const int64_t head_row0 = (int64_t)h * a.T;   // the head's first row in the workspace
  // the state: S[16 dt + 4 g + x][col] in Sreg[dt][x]
  gla_f32x4 Sreg[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int d = 16 * dt + 4 * g + x;
      Sreg[dt][x] = has_col && d < dim ? st[(int64_t)d * vdim + col] : 0.f;
    }
  const gla_f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  // The loads of a chunk's operands, every one of them unconditional (a load inside a branch is
  // waited for where the branch ends): rows, channels and columns beyond the last are fetched
  // from the last, a chunk beyond the last from the last, and `chunk` puts zeros where they count.
  const int last_chunk = n > 0 ? (n - 1) / kGlaChunk * kGlaChunk : 0;
  const int col_c = min(col, vdim - 1);
  auto fetch = [&](GlaChunkRegs<DT>& R, int i0) {
    i0 = min(i0, last_chunk);
    const int L = min(kGlaChunk, n - i0), base = r0 + i0;
    const float* qrow = a.qe + (head_row0 + base + min(c, L - 1)) * dim;
    const float* erow = a.eb + (head_row0 + base + L - 1) * dim;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int d = min(16 * dt + 4 * g, dim - 4);   // (dim is a multiple of 4)
      R.q[dt] = *(const gla_f32x4*)(qrow + d);
      R.e[dt] = *(const gla_f32x4*)(erow + d);
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int64_t row = base + min(4 * g + x, L - 1);
      const float* krow = a.ke + (head_row0 + row) * dim;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) R.k[x][dt] = krow[min(16 * dt + c, dim - 1)];
      R.v[x] = to_f32(((const T*)a.g.qkv)[row * a.g.stride + a.g.v_off + h * vdim + col_c]);
    }
    R.A = *(const gla_f32x4*)(a.A + (head_row0 + base + min(c, L - 1)) * kGlaChunk + 4 * g);
  };
  // a chunk: its outputs from the state before it, then the state after it; the operands of the
  // chunk after the next one set out first (three sets of registers take turns)
  auto chunk = [&](GlaChunkRegs<DT>& cur, int i0, GlaChunkRegs<DT>& ahead) {
    const int L = min(kGlaChunk, n - i0);
    fetch(ahead, i0 + 2 * kGlaChunk);
    // zeros where a sum runs over rows or channels that are not there
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (16 * dt + 4 * g >= dim) cur.q[dt] = zero4, cur.e[dt] = zero4;
#pragma unroll
      for (int x = 0; x < 4; ++x)
        if (4 * g + x >= L || 16 * dt + c >= dim) cur.k[x][dt] = 0.f;
    }
#pragma unroll
    for (int x = 0; x < 4; ++x)
      if (4 * g + x >= L) cur.v[x] = 0.f;
    // the outputs: rows 4 g + x of column c in o[x] + o2[x]
    gla_f32x4 o = zero4, o2 = zero4;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      o = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.q[dt][0], Sreg[dt][0], o, 0, 0, 0);
      o2 = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.q[dt][1], Sreg[dt][1], o2, 0, 0, 0);
      o = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.q[dt][2], Sreg[dt][2], o, 0, 0, 0);
      o2 = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.q[dt][3], Sreg[dt][3], o2, 0, 0, 0);
    }
    o = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.A[0], cur.v[0], o, 0, 0, 0);
    o2 = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.A[1], cur.v[1], o2, 0, 0, 0);
    o = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.A[2], cur.v[2], o, 0, 0, 0);
    o2 = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.A[3], cur.v[3], o2, 0, 0, 0);
    if (has_col) {
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int t = 4 * g + x;
        if (t < L) a.g.out[((int64_t)(r0 + i0 + t) * H + h) * vdim + col] = o[x] + o2[x];
      }
    }
    // the state after the chunk
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int x = 0; x < 4; ++x) Sreg[dt][x] *= cur.e[dt][x];
#pragma unroll
      for (int x = 0; x < 4; ++x)
        Sreg[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.k[x][dt], cur.v[x], Sreg[dt], 0, 0, 0);
    }
  };
  GlaChunkRegs<DT> R0, R1, R2;
  if (n <= 0) return;
  fetch(R0, 0);
  fetch(R1, kGlaChunk);
  for (int i0 = 0; i0 < n; i0 += 3 * kGlaChunk) {
    chunk(R0, i0, R2);
    if (i0 + kGlaChunk >= n) break;
    chunk(R1, i0 + kGlaChunk, R0);
    if (i0 + 2 * kGlaChunk >= n) break;
    chunk(R2, i0 + 2 * kGlaChunk, R1);
  }
  if (has_col) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int d = 16 * dt + 4 * g + x;
        if (d < dim) st[(int64_t)d * vdim + col] = Sreg[dt][x];
      }
  }
}

}  // namespace ninfer

// The same as ninfer_gated_linear_attention for bfloat16 rows, in chunks of 16 rows on the
// matrix cores: for steps that bring prompt portions. `work` holds T * (3 heads dim + 16 heads)
// floats. Returns 1 (nothing launched) when the sizes do not fit.
extern "C" int ninfer_gated_linear_attention_chunks(const void* qkv, int stride, int q_off, int k_off,
                                                    int v_off, const float* z, float tau,
                                                    float q_scale, float* state,
                                                    long long state_stride, float* out,
                                                    const int* seq_row_start, const int* seq_slots,
                                                    float* work, int T, int S, int H, int dim,
                                                    int vdim, int dtype, hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && S > 0 && H > 0 && dim > 0 && vdim > 0,
                 "gated_linear_attention: T=%d S=%d heads=%d dim=%d vdim=%d must be positive", T,
                 S, H, dim, vdim);
  NINFER_REQUIRE(tau > 0.f, "gated_linear_attention: tau (%g) must be positive", tau);
  NINFER_REQUIRE(state_stride >= (long long)H * dim * vdim,
                 "gated_linear_attention: a request's state of %lld floats holds no %d x %d x %d",
                 state_stride, H, dim, vdim);
  NINFER_REQUIRE(work != nullptr, "gated_linear_attention: the chunks need their workspace");
  if (dtype != kBF16 || dim > kGlaChunkMaxDim || dim % 4 != 0 || (uintptr_t)work % 16 != 0) return 1;
  GlaChunkArgs a;
  a.g.qkv = qkv, a.g.z = z, a.g.state = state, a.g.out = out;
  a.g.seq_row_start = seq_row_start, a.g.seq_slots = seq_slots, a.g.state_stride = state_stride;
  a.g.stride = stride, a.g.q_off = q_off, a.g.k_off = k_off, a.g.v_off = v_off;
  a.g.H = H, a.g.dim = dim, a.g.vdim = vdim, a.g.inv_tau = 1.f / tau, a.g.q_scale = q_scale;
  const int64_t thd = (int64_t)T * H * dim;
  a.qe = work, a.ke = work + thd, a.eb = work + 2 * thd, a.A = work + 3 * thd;
  a.T = T, a.S = S;
  const int chunks = T / kGlaChunk + S;   // no step has more: each request adds at most one short chunk
  gla_chunk_prepare_kernel<bf16><<<dim3(chunks, H), 256, 0, stream>>>(a);
  const int cols = kGlaCols * kGlaWaves;
  const dim3 grid(S, H, (vdim + cols - 1) / cols);
  if (dim <= 16) gla_chunk_scan_kernel<bf16, 1><<<grid, 64 * kGlaWaves, 0, stream>>>(a);
  else if (dim <= 32) gla_chunk_scan_kernel<bf16, 2><<<grid, 64 * kGlaWaves, 0, stream>>>(a);
  else if (dim <= 64) gla_chunk_scan_kernel<bf16, 4><<<grid, 64 * kGlaWaves, 0, stream>>>(a);
  else gla_chunk_scan_kernel<bf16, 8><<<grid, 64 * kGlaWaves, 0, stream>>>(a);
  NINFER_LAUNCH_CHECK();
  return 0;
}
