// Attention without a softmax on the matrix cores (bf16 rows and cache; see
// attention_sigmoid.h for what it computes).
//
// A block of eight waves owns a tile of 32 rows of one request with all heads (and, of values
// wider than 128, one part of the columns), and every
// n_splits-th tile of 32 keys of the range those rows can see (weights are not normalised over
// keys, so the parts of a row's output over disjoint keys simply add: with more than one
// split they go to a 32-bit workspace and a second kernel adds them in a fixed order). All
// heads meet in one block because the mixing of the heads' weights needs every head's weight
// of a (row, key) pair at once.
//
// A tile of keys and values of all kv heads goes global memory -> registers (one tile ahead)
// -> LDS (one buffer). Wave w looks after the heads w, w + 8, ... (HPW of them). With
// v_mfma_f32_32x32x16_bf16 it computes for each of its heads
//   S^T[key][row] = K Q^T          (A = key rows from LDS, B = the head's queries, fetched again for every tile)
// whose accumulators give lane l the scores of row l % 32 for the keys 8 (v / 4) + 4 (l / 32)
// + v % 4; scale, bias, sigmoid and the mask run on them in 32-bit, and the weights go to LDS
// lane by lane ([head][v][lane]: a lane holds the same (row, key) pairs in every wave). After a
// barrier wave w forms, for the pairs (v = 2 w, 2 w + 1; every lane) and every head a,
//   w'_a = sum_b mix[a, b] w_b     (32-bit; the matrix from LDS, padded with zeros to 8 HPW
//                                   heads so that the sums have no branch)
// in the places of the plain weights: a weight is read once, not once per head. After another
// barrier a wave reads its heads' weights (mixed or not) back,
// which, rounded to bf16, is the B operand of
//   O^T[value column][row] += V^T W'^T   (A = V^T: the transposing LDS read hands a lane four
//                                         consecutive keys of one value column)
// Keys that do not exist (beyond the tile's last row) load the last row's key in their place:
// they are masked, and their values must be finite since 0 x NaN is not 0.
#include "attention_sigmoid.h"

namespace ninfer {

typedef __bf16 sg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float sg_f32x16 __attribute__((ext_vector_type(16)));
typedef short sg_short4 __attribute__((ext_vector_type(4)));
typedef short sg_short8 __attribute__((ext_vector_type(8)));
typedef unsigned int sg_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) sg_short4 sg_lds_short4;

constexpr int kSgWaves = 8;
constexpr int kSgThreads = 64 * kSgWaves;
constexpr int kSgKeys = 32;          // keys per tile
constexpr int kSgRows = 32;          // rows per tile
// 32-column blocks of the values that a block of threads looks after (the block's z index
// chooses among the parts of wider values)
static inline int sg_db(int vdim) { return vdim <= 64 ? 2 : 4; }
constexpr int kSgPieces = 4;         // 16-byte pieces of a key (value) tile per thread
constexpr float kSgLog2e = 1.44269504088896f;

// Which request and which of its row tiles is tile `idx` (counted from the step's last)?
__device__ __forceinline__ bool sg_find_tile(const SigAttnArgs& a, int idx, int* seq, int* row0,
                                             int* n_rows) {
  if (a.max_qlen == 1) {   // every request brings one row, which is a tile
    if (idx >= a.S) return false;
    *seq = a.S - 1 - idx, *row0 = *seq, *n_rows = 1;
    return true;
  }
  for (int s = a.S - 1; s >= 0; --s) {
    const int b = a.seq_row_start[s], e = a.seq_row_start[s + 1];
    const int nt = (e - b + kSgRows - 1) / kSgRows;
    if (idx < nt) {
      *seq = s;
      *row0 = b + (nt - 1 - idx) * kSgRows;   // a request's last row tiles walk the most keys: first
      *n_rows = min(kSgRows, e - *row0);
      return true;
    }
    idx -= nt;
  }
  return false;
}

template <int KS, int DB, int HPW>
__global__ __launch_bounds__(kSgThreads) void sigmoid_attention_tiles_kernel(SigAttnArgs a,
                                                                           float* part,
                                                                           int n_splits) {
  constexpr int DP = 16 * KS, KROW = DP + 8, VP = 32 * DB, VROW = VP + 8;
  extern __shared__ __attribute__((aligned(16))) unsigned short lds[];
  const int G = a.Hkv, H = a.Hq, hpg = H / G;
  unsigned short* k_s = lds;                               // [G][32 keys][KROW]
  unsigned short* v_s = k_s + G * kSgKeys * KROW;          // [G][32 keys][VROW]
  float* w_s = (float*)(v_s + G * kSgKeys * VROW);         // [H][16][64]
  constexpr int MAXH = kSgWaves * HPW;
  float* m_s = w_s + H * 16 * 64;                          // [MAXH][MAXH] the mixing matrix, zeros beyond H

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, hi = lane >> 5;
  int seq, row0, n_rows;
  if (!sg_find_tile(a, blockIdx.x, &seq, &row0, &n_rows)) return;
  const int split = blockIdx.y;
  // the block's part of the value columns (a head's output over all of them at once would need
  // more accumulators than a wave has registers for): 32 DB columns from vbase on
  const int vbase = VP * blockIdx.z, vwidth = min(VP, a.vdim - vbase);
  const int pos_first = a.positions[row0], pos_last = pos_first + n_rows - 1;
  const int key_first = a.chunk > 0 ? pos_first / a.chunk * a.chunk : 0;
  const int* bt = a.block_table + (int64_t)seq * a.bt_stride;
  const int ps_shift = __builtin_ctz(a.page_size), ps_mask = a.page_size - 1;
  const int dim = a.dim, vdim = a.vdim;
  const unsigned short* kpool = (const unsigned short*)a.kpool;
  const unsigned short* vpool = (const unsigned short*)a.vpool;

  // zeros everywhere once: the padding columns stay zero, the rest is overwritten
  {
    const int n16 = G * kSgKeys * (KROW + VROW) / 8;
    for (int i = tid; i < n16; i += kSgThreads) ((sg_u32x4*)lds)[i] = sg_u32x4{0u, 0u, 0u, 0u};
  }

  if (a.mix)
    for (int i = tid; i < MAXH * MAXH; i += kSgThreads) {
      const int ma = i / MAXH, mb = i % MAXH;
      m_s[i] = ma < H && mb < H ? a.mix[ma * H + mb] : 0.f;
    }

  // this thread's pieces of a tile (16 bytes each): kv head, key, column. Every load is
  // unconditional: a piece that does not exist loads the tile's last piece once more and is
  // not stored.
  int k_g[kSgPieces], k_key[kSgPieces], k_col[kSgPieces], v_g[kSgPieces], v_key[kSgPieces], v_col[kSgPieces];
  bool k_ok[kSgPieces], v_ok[kSgPieces];
  {
    const int cpk = dim / 8, cpv = vwidth / 8;
    const int nk = G * kSgKeys * cpk, nv = G * kSgKeys * cpv;
#pragma unroll
    for (int i = 0; i < kSgPieces; ++i) {
      const int p = i * kSgThreads + tid;
      k_ok[i] = p < nk;
      const int pk = min(p, nk - 1);
      k_g[i] = pk / (kSgKeys * cpk);
      k_key[i] = pk / cpk % kSgKeys;
      k_col[i] = pk % cpk * 8;
      v_ok[i] = p < nv;
      const int pv = min(p, nv - 1);
      v_g[i] = pv / (kSgKeys * cpv);
      v_key[i] = pv / cpv % kSgKeys;
      v_col[i] = pv % cpv * 8;
    }
  }
  sg_u32x4 kreg[kSgPieces], vreg[kSgPieces];
  // The pages of a tile's pieces are looked up a tile before the pieces are fetched: a wave
  // issues its instructions in order, and a fetch whose address waits for the block table's
  // entry would hold up everything behind it.
  int k_page[kSgPieces], v_page[kSgPieces];
#define NINFER_SIG_LOOK_UP(K0)                                                                       \
  {                                                                                                  \
    _Pragma("unroll") for (int i = 0; i < kSgPieces; ++i) {                                          \
      k_page[i] = bt[min((K0) + k_key[i], pos_last) >> ps_shift];                                    \
      v_page[i] = bt[min((K0) + v_key[i], pos_last) >> ps_shift];                                    \
    }                                                                                                \
  }
#define NINFER_SIG_LOAD_TILE(K0)                                                                     \
  {                                                                                                  \
    _Pragma("unroll") for (int i = 0; i < kSgPieces; ++i) {                                          \
      const int j = min((K0) + k_key[i], pos_last);                                                  \
      const int64_t at = ((int64_t)k_page[i] * G + k_g[i]) * a.page_size + (j & ps_mask);            \
      kreg[i] = *(const sg_u32x4*)(kpool + at * dim + k_col[i]);                                     \
    }                                                                                                \
    _Pragma("unroll") for (int i = 0; i < kSgPieces; ++i) {                                          \
      const int j = min((K0) + v_key[i], pos_last);                                                  \
      const int64_t at = ((int64_t)v_page[i] * G + v_g[i]) * a.page_size + (j & ps_mask);            \
      vreg[i] = *(const sg_u32x4*)(vpool + at * vdim + vbase + v_col[i]);                           \
    }                                                                                                \
    NINFER_SIG_LOOK_UP((K0) + n_splits * kSgKeys)                                                    \
  }
#define NINFER_SIG_STORE_TILE()                                                                      \
  {                                                                                                  \
    _Pragma("unroll") for (int i = 0; i < kSgPieces; ++i) {                                          \
      if (k_ok[i]) *(sg_u32x4*)(k_s + (k_g[i] * kSgKeys + k_key[i]) * KROW + k_col[i]) = kreg[i];    \
      if (v_ok[i]) *(sg_u32x4*)(v_s + (v_g[i] * kSgKeys + v_key[i]) * VROW + v_col[i]) = vreg[i];    \
    }                                                                                                \
  }

  // this lane's queries (B operand): row c of the tile, dims 16 ks + 8 hi .. + 7 of each of the
  // wave's heads
  const bool q_valid = c < n_rows;
  const int q_pos = pos_first + c;
  const int q_first = a.chunk > 0 ? q_pos / a.chunk * a.chunk : 0;   // the first key the row sees
  // (fetched again for every tile of keys, from the cache: kept in registers beside the
  // outputs' accumulators they would not fit, and what does not fit goes to scratch memory)
  unsigned q_at[HPW];   // where row c of the wave's head i begins, in numbers from a.qkv on
  float bias2[HPW];
  bool head_ok[HPW];
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    const int h = wave + kSgWaves * i;
    head_ok[i] = h < H;
    const int hh = head_ok[i] ? h : 0;
    bias2[i] = a.head_bias ? a.head_bias[hh] * kSgLog2e : 0.f;
    q_at[i] = (unsigned)((row0 + (q_valid ? c : 0)) * a.q_stride + hh * dim);
  }
  const float scale2 = a.scale * kSgLog2e;

  sg_f32x16 o[HPW][DB];
#pragma unroll
  for (int i = 0; i < HPW; ++i)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[i][db][v] = 0.f;

  // the transposing read's address of this lane inside a value tile: lane s of a group of 16
  // fetches key s / 4 (+ 4 hi), value columns 16 (group % 2) + 4 (s % 4) .. + 3
  const int s16 = lane & 15, q4 = lane >> 4;
  const int v_lane = (4 * hi + s16 / 4) * VROW + 16 * (q4 & 1) + 4 * (s16 & 3);

  const int t_first = key_first / kSgKeys + split, t_end = pos_last / kSgKeys + 1;
  NINFER_SIG_LOOK_UP(t_first * kSgKeys)
  if (t_first < t_end) NINFER_SIG_LOAD_TILE(t_first * kSgKeys)
  __syncthreads();   // the zeros are written
  for (int kt = t_first; kt < t_end; kt += n_splits) {
    const int k0 = kt * kSgKeys;
    NINFER_SIG_STORE_TILE()
    __syncthreads();   // the tile is in LDS
    if (kt + n_splits < t_end) NINFER_SIG_LOAD_TILE(k0 + n_splits * kSgKeys)
    // some row of the tile does not see every key of this tile
    const bool masked = k0 + kSgKeys - 1 > pos_first || k0 < (a.chunk > 0 ? pos_last / a.chunk * a.chunk : 0);
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      if (!head_ok[i]) continue;
      const int h = wave + kSgWaves * i, g = h / hpg;
      const unsigned short* kg = k_s + g * kSgKeys * KROW;
      sg_f32x16 s;
#pragma unroll
      for (int v = 0; v < 16; ++v) s[v] = 0.f;
      // this lane's queries (B operand): row c of the tile, dims 16 ks + 8 hi .. + 7 (a part
      // beyond dim loads the last part and counts as zeros; a row that is not there loads the
      // tile's first, and its outputs are not stored)
      unsigned qa = q_at[i];
      asm volatile("" : "+v"(qa));   // (not to be moved out of the loop)
      const unsigned short* qr = (const unsigned short*)a.qkv + qa;
      sg_u32x4 qv[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qv[ks] = *(const sg_u32x4*)(qr + min(16 * ks + 8 * hi, dim - 8));
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const sg_bf16x8 kf = *(const sg_bf16x8*)(kg + c * KROW + 16 * ks + 8 * hi);
        if (16 * ks + 8 * hi >= dim) qv[ks] = sg_u32x4{0u, 0u, 0u, 0u};
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, __builtin_bit_cast(sg_bf16x8, qv[ks]), s, 0, 0, 0);
      }
      float* wh = w_s + (h * 16) * 64 + lane;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        // sigmoid(x) = 1 / (1 + 2^(-x log2 e))
        float w = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-(s[v] * scale2 + bias2[i])));
        if (masked) {
          const int kp = k0 + 8 * (v >> 2) + 4 * hi + (v & 3);
          if (kp > q_pos || kp < q_first) w = 0.f;
        }
        wh[v * 64] = w;
      }
    }
    __syncthreads();   // every head's weights are in LDS
    if (a.mix) {
      // w'_a = sum_b mix[a, b] w_b. Wave w does it for the pairs (v = 2 w, 2 w + 1; every lane)
      // and all heads, so that a weight is read from LDS once, not once per head; the mixed
      // weights take the places of the plain ones (no other wave reads or writes these pairs
      // in this phase, and the wave has read all of them before it writes the first).
      // (no branch inside the sums: a load behind a branch is waited for at once)
      float w0[MAXH], w1[MAXH];
#pragma unroll
      for (int b = 0; b < MAXH; ++b) {
        const int bb = min(b, H - 1);   // heads that are not there: some head's weight times zero
        w0[b] = w_s[(bb * 16 + 2 * wave) * 64 + lane];
        w1[b] = w_s[(bb * 16 + 2 * wave + 1) * 64 + lane];
      }
#pragma unroll
      for (int aa = 0; aa < MAXH; ++aa) {
        if (aa >= H) break;
        const float* mrow = m_s + aa * MAXH;
        float m0 = 0.f, m1 = 0.f;
#pragma unroll
        for (int b = 0; b < MAXH; ++b) {
          const float tb = mrow[b];
          m0 = fmaf(tb, w0[b], m0);
          m1 = fmaf(tb, w1[b], m1);
        }
        w_s[(aa * 16 + 2 * wave) * 64 + lane] = m0;
        w_s[(aa * 16 + 2 * wave + 1) * 64 + lane] = m1;
      }
      __syncthreads();   // every head's mixed weights are in LDS
    }
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      if (!head_ok[i]) continue;
      const int h = wave + kSgWaves * i, g = h / hpg;
      sg_bf16x8 pf[2];
      const float* wb = w_s + (h * 16) * 64 + lane;
#pragma unroll
      for (int v = 0; v < 16; ++v) pf[v >> 3][v & 7] = (__bf16)wb[v * 64];
      const unsigned short* vg = v_s + g * kSgKeys * VROW;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          const unsigned short* p = vg + v_lane + 16 * hh * VROW + 32 * db;
          const sg_short4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((sg_lds_short4*)p);
          const sg_short4 up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((sg_lds_short4*)(p + 8 * VROW));
          sg_short8 both;
          both.s0 = lo.x; both.s1 = lo.y; both.s2 = lo.z; both.s3 = lo.w;
          both.s4 = up.x; both.s5 = up.y; both.s6 = up.z; both.s7 = up.w;
          o[i][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(sg_bf16x8, both), pf[hh],
                                                            o[i][db], 0, 0, 0);
        }
    }
    __syncthreads();   // the tile and the weights are read: the next may overwrite them
  }
  // Lane holds, for row c, value columns 32 db + 8 (v / 4) + 4 hi + v % 4 of each of its heads.
  if (!q_valid) return;
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    if (!head_ok[i]) continue;
    const int h = wave + kSgWaves * i;
    const int64_t at = ((int64_t)(row0 + c) * H + h) * vdim;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        if (32 * db + 8 * v4 + 4 * hi >= vwidth) continue;   // value sizes are multiples of 8: four columns are there together
        const int col = vbase + 32 * db + 8 * v4 + 4 * hi;
        if (part) {
          float* pr = part + (int64_t)split * a.T * H * vdim + at + col;
          *(float4*)pr = make_float4(o[i][db][4 * v4], o[i][db][4 * v4 + 1], o[i][db][4 * v4 + 2],
                                     o[i][db][4 * v4 + 3]);
        } else {
          union { __bf16 b[4]; uint2 u; } w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w.b[e] = (__bf16)o[i][db][4 * v4 + e];
          *(uint2*)((unsigned short*)a.out + at + col) = w.u;
        }
      }
  }
}

// out[t, e] = sum over the splits, in their order.
__global__ void sigmoid_attention_sum_kernel(const float* __restrict__ part, __hip_bfloat16* __restrict__ out,
                                             int64_t n, int n_splits) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= n) return;
  float4 s = *(const float4*)(part + i);
  for (int k = 1; k < n_splits; ++k) {
    const float4 x = *(const float4*)(part + k * n + i);
    s.x += x.x, s.y += x.y, s.z += x.z, s.w += x.w;
  }
  union { __bf16 b[4]; uint2 u; } w;
  w.b[0] = (__bf16)s.x, w.b[1] = (__bf16)s.y, w.b[2] = (__bf16)s.z, w.b[3] = (__bf16)s.w;
  *(uint2*)((unsigned short*)out + i) = w.u;
}

// LDS of a block: the tile of keys and values, every head's weights in 32-bit and the mixing
// matrix.
static size_t sg_lds_bytes(const SigAttnArgs& a, int krow, int vrow) {
  return (size_t)a.Hkv * kSgKeys * (krow + vrow) * sizeof(unsigned short) +
         (size_t)a.Hq * 16 * 64 * sizeof(float) + (size_t)4 * kSgWaves * kSgWaves * sizeof(float);
}

bool sigmoid_attention_tiles_takes(const SigAttnArgs& a) {
  return sg_lds_bytes(a, 16 * (a.dim <= 64 ? 4 : 8) + 8, 32 * sg_db(a.vdim) + 8) <= 160 * 1024 &&
         (int64_t)a.T * a.q_stride < (1ll << 31) && a.dtype == kBF16 && a.dim % 8 == 0 && a.vdim % 8 == 0 && a.dim <= 128 && a.vdim <= 128 &&
         a.q_stride % 8 == 0 && (a.page_size & (a.page_size - 1)) == 0 && a.Hq <= 2 * kSgWaves &&
         a.Hkv * kSgKeys * (a.dim / 8) <= kSgPieces * kSgThreads &&
         a.Hkv * kSgKeys * (min(a.vdim, 32 * sg_db(a.vdim)) / 8) <= kSgPieces * kSgThreads;
}

// Into how many parts are the keys cut, so that the launch fills the GPU? A row tile walks at
// most (visible keys) / 32 key tiles; `tiles` row tiles are launched.
int sigmoid_attention_tiles_splits(const SigAttnArgs& a) {
  const int tiles = (a.max_qlen == 1 ? a.T : (a.T + kSgRows - 1) / kSgRows + a.S / 2) *
                    ((a.vdim + 32 * sg_db(a.vdim) - 1) / (32 * sg_db(a.vdim)));
  const int span = a.chunk > 0 ? min(a.chunk + kSgRows, a.max_kv_len) : a.max_kv_len;
  const int key_tiles = (span + kSgKeys - 1) / kSgKeys + 1;
  int want = (2 * device_cu_count() + tiles - 1) / tiles;
  if (want > key_tiles) want = key_tiles;
  if (want > 64) want = 64;
  return want < 1 ? 1 : want;
}

template <int KS, int DB, int HPW>
static int launch_sig_tiles(const SigAttnArgs& a, float* part, int n_splits, hipStream_t stream) {
  constexpr int KROW = 16 * KS + 8, VP = 32 * DB, VROW = VP + 8;
  const size_t lds = sg_lds_bytes(a, KROW, VROW);
  auto kern = sigmoid_attention_tiles_kernel<KS, DB, HPW>;
  if (lds > 64 * 1024) {
    static size_t raised = 0;   // per instantiation
    if (lds > raised) {
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return set_error(-2, "sigmoid_attention: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
      raised = lds;
    }
  }
  // an upper bound of the row tiles: every request may end with a partly filled one
  const int tiles = a.max_qlen == 1 ? a.T : a.T / kSgRows + a.S;
  kern<<<dim3(tiles, n_splits, (a.vdim + VP - 1) / VP), kSgThreads, lds, stream>>>(a, part, n_splits);
  NINFER_LAUNCH_CHECK();
  if (part) {
    const int64_t n = (int64_t)a.T * a.Hq * a.vdim;
    sigmoid_attention_sum_kernel<<<(unsigned)((n / 4 + 255) / 256), 256, 0, stream>>>(
        part, (__hip_bfloat16*)a.out, n, n_splits);
    NINFER_LAUNCH_CHECK();
  }
  return 0;
}

// `part`: 32-bit scratch of n_splits x T x Hq x vdim numbers when n_splits > 1, else null.
int sigmoid_attention_tiles(const SigAttnArgs& a, float* part, int n_splits, hipStream_t stream) {
  const int ks = a.dim <= 64 ? 4 : 8;
  const int hpw = a.Hq <= kSgWaves ? 1 : 2;
  if (n_splits <= 1) part = nullptr;
#define NINFER_SIG_TILES(KS_, DB_)                                                          \
  return hpw == 1 ? launch_sig_tiles<KS_, DB_, 1>(a, part, n_splits, stream)                \
                  : launch_sig_tiles<KS_, DB_, 2>(a, part, n_splits, stream)
  const int db = sg_db(a.vdim);
  if (ks == 4 && db == 2) NINFER_SIG_TILES(4, 2);
  if (ks == 4) NINFER_SIG_TILES(4, 4);
  if (db == 2) NINFER_SIG_TILES(8, 2);
  NINFER_SIG_TILES(8, 4);
#undef NINFER_SIG_TILES
}

}  // namespace ninfer
