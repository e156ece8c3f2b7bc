// Attention over a cached latent: every head reads the same cached row per key,
// [c (R numbers) | k_rot (rd numbers)], and a query that has been taken into the latent's
// space, q' = [W_uk_h^T q_unrotated (R) | q_rotated (rd)]:
//
//   score_j = (q' . row_j) * scale,  p = softmax over the visible keys,  o = sum_j p_j c_j
//
// so that neither keys nor values per head are ever formed for the cache: the head's value
// is W_uv_h o afterwards. Two kernels:
//
//   latent_kv_write  per row: c = rmsnorm(first R of the down-projection) * weight, the
//                    shared rotated key part turned by the row's position, both written to
//                    the request's page; the rotated part of every query head turned and
//                    placed behind the R absorbed numbers of q'.
//   latent_attention one wave per (row, head); keys in tiles of 64 aligned to absolute
//                    positions with an online softmax, so every sum's order depends on the
//                    row's position alone. The head's output may be multiplied by
//                    sigmoid(gate[row, head]).
//
//   latent_attention_tile (bfloat16, matrix cores): a block of four waves owns 32 rows of
//                    (token, head) pairs of one request, all of which read the same cached
//                    rows. Keys come in tiles of 64 through LDS as they lie in the cache
//                    ([key][numbers]); S = Q' K^T and O += P V run on v_mfma_f32_32x32x16_bf16,
//                    the softmax between them in 32-bit on eight lanes per row. The value
//                    operand needs eight keys of one column per lane and takes them from
//                    the tile by eight two-byte LDS reads. The keys of long contexts are cut
//                    into chunks over several blocks whose partial sums a second kernel
//                    merges (steps of few rows would otherwise leave most of the GPU idle).
//
// The rotation turns pair (i, i + n/2), or with `interleaved` pair (2i, 2i + 1), of the first
// n = rot_n numbers of the rotated part by pos * freq[i]; cosine and sine are multiplied by `magnitude` (1 without a scaled table).
// Norm, angles, scores, softmax and the value sum are 32-bit.
#include "common.h"

namespace ninfer {

struct LatentArgs {
  const void* dkv;          // [T, dkv_stride] down-projection rows: R latent numbers, then rd
  const void* q;            // [T, Hq * (dim + rd)] projected queries, head by head
  float* q_abs;             // [T, Hq, R + rd] 32-bit; the first R of each head are written by
                            // the caller's products, the last rd here
  void* pool;               // [pages, page_size, R + rd]
  void* out;                // [T, Hq * R] (attention) in the activation dtype
  const void* gate;         // [T, gate_stride] or null: out of head h times sigmoid(gate[t, h])
  const float* norm_w;      // [R]
  const float* freq;        // [rot_n / 2]
  const int* block_table;   // [S, bt_stride]
  const int* positions;     // [T]
  const int* row_seq;       // [T]
  const int* seq_row_start; // [S + 1] (the matrix-core kernel: rows of each request)
  const int* seq_pos0;      // [S] position of each request's first row
  float* workspace;         // partial sums of contexts cut into chunks, or null
  long long workspace_floats;
  int S;
  int max_kv_len;           // host-side bound that sizes the chunks
  int max_qlen;             // host-side: the most rows a request brings (1: a decode-only step)
  int force_plain;          // tests: the plain kernel whatever the shape
  int dkv_stride;
  int gate_stride;
  int bt_stride;
  int T;
  int Hq;
  int dim;                  // unrotated numbers per query head
  int R;                    // latent size
  int rd;                   // rotated numbers per head (and of the shared key part)
  int rot_n;                // how many of them turn (even, <= rd)
  int page_size;
  int window;               // 0: all keys
  int write_kv;
  int dtype;
  float eps;
  float magnitude;
  float scale;
  int interleaved;          // pair i of the turning numbers is (2i, 2i + 1) instead of (i, i + rot_n / 2)
};

__device__ __forceinline__ void turn_pair(float u, float v, float c, float s, float* a, float* b) {
  *a = u * c - v * s;
  *b = v * c + u * s;
}

template <typename T>
__global__ void latent_kv_write_kernel(LatentArgs a) {
  extern __shared__ float smem[];
  float* trig = smem;            // [rot_n]: cos, then sin
  __shared__ float red[16];
  const int t = blockIdx.x;
  const int pos = a.positions[t];
  const int half = a.rot_n / 2;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float s, c;
    sincosf((float)pos * a.freq[i], &s, &c);
    trig[i] = c * a.magnitude;
    trig[half + i] = s * a.magnitude;
  }
  const T* row = (const T*)a.dkv + (int64_t)t * a.dkv_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < a.R; i += blockDim.x) {
    const float v = to_f32(row[i]);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, red);   // (its barriers also publish trig)
  const int Dk = a.R + a.rd;
  if (a.write_kv) {
    const float inv = 1.f / sqrtf(ss / (float)a.R + a.eps);
    const int page = a.block_table[(int64_t)a.row_seq[t] * a.bt_stride + pos / a.page_size];
    T* dst = (T*)a.pool + ((int64_t)page * a.page_size + pos % a.page_size) * Dk;
    for (int i = threadIdx.x; i < a.R; i += blockDim.x)
      dst[i] = from_f32<T>(to_f32(row[i]) * inv * a.norm_w[i]);
    const T* kr = row + a.R;
    for (int i = threadIdx.x; i < a.rd; i += blockDim.x) {
      float v = to_f32(kr[i]);
      if (i < a.rot_n) {
        const int p = a.interleaved ? i >> 1 : i < half ? i : i - half;
        const int i1 = a.interleaved ? 2 * p : p, i2 = a.interleaved ? 2 * p + 1 : p + half;
        float x, y;
        turn_pair(to_f32(kr[i1]), to_f32(kr[i2]), trig[p], trig[half + p], &x, &y);
        v = i == i1 ? x : y;
      }
      dst[a.R + i] = from_f32<T>(v);
    }
  }
  const int qd = a.dim + a.rd;
  for (int e = threadIdx.x; e < a.Hq * a.rd; e += blockDim.x) {
    const int h = e / a.rd, i = e % a.rd;
    const T* qr = (const T*)a.q + ((int64_t)t * a.Hq + h) * qd + a.dim;
    float v = to_f32(qr[i]);
    if (i < a.rot_n) {
      const int p = a.interleaved ? i >> 1 : i < half ? i : i - half;
      const int i1 = a.interleaved ? 2 * p : p, i2 = a.interleaved ? 2 * p + 1 : p + half;
      float x, y;
      turn_pair(to_f32(qr[i1]), to_f32(qr[i2]), trig[p], trig[half + p], &x, &y);
      v = i == i1 ? x : y;
    }
    a.q_abs[((int64_t)t * a.Hq + h) * Dk + a.R + i] = v;
  }
}

constexpr int kLatentMaxPerLane = 16;   // latent sizes up to 1024

template <typename T>
__global__ __launch_bounds__(64) void latent_attention_kernel(LatentArgs a) {
  extern __shared__ float smem[];
  const int Dk = a.R + a.rd;
  int64_t* off_s = (int64_t*)smem;         // [64] element offset of each key's row
  float* p_s = (float*)(off_s + 64);       // [64]
  float* q_s = p_s + 64;                   // [Dk]
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int pos = a.positions[t];
  const int* bt = a.block_table + (int64_t)a.row_seq[t] * a.bt_stride;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const float* qr = a.q_abs + ((int64_t)t * a.Hq + h) * Dk;
  for (int d = lane; d < Dk; d += 64) q_s[d] = qr[d];
  __syncthreads();
  const T* pool = (const T*)a.pool;
  float m = -INFINITY, l = 0.f;
  float acc[kLatentMaxPerLane];
#pragma unroll
  for (int i = 0; i < kLatentMaxPerLane; ++i) acc[i] = 0.f;
  for (int tile = (lo / 64) * 64; tile <= pos; tile += 64) {
    const int j = tile + lane;
    const bool valid = j >= lo && j <= pos;
    float s = -INFINITY;
    int64_t off = 0;
    if (valid) {
      const int page = bt[j / a.page_size];
      off = ((int64_t)page * a.page_size + (j % a.page_size)) * Dk;
      const T* kr = pool + off;
      float dot = 0.f;
      for (int d = 0; d < Dk; ++d) dot = fmaf(q_s[d], to_f32(kr[d]), dot);
      s = dot * a.scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);   // 0 on the first tile
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[lane] = p;
    off_s[lane] = off;
    __syncthreads();
    const int n_keys = min(64, pos - tile + 1);
    const int first = max(0, lo - tile);
#pragma unroll
    for (int i = 0; i < kLatentMaxPerLane; ++i) {
      const int d = lane + i * 64;
      if (d < a.R) {
        float v = acc[i] * alpha;
        for (int jj = first; jj < n_keys; ++jj) v = fmaf(p_s[jj], to_f32(pool[off_s[jj] + d]), v);
        acc[i] = v;
      }
    }
    __syncthreads();
  }
  float inv = 1.f / l;
  if (a.gate) {
    const float g = to_f32(((const T*)a.gate)[(int64_t)t * a.gate_stride + h]);
    inv *= 1.f / (1.f + expf(-g));
  }
  T* orow = (T*)a.out + ((int64_t)t * a.Hq + h) * a.R;
#pragma unroll
  for (int i = 0; i < kLatentMaxPerLane; ++i) {
    const int d = lane + i * 64;
    if (d < a.R) orow[d] = from_f32<T>(acc[i] * inv);
  }
}

static bool latent_tile_takes(const LatentArgs& a);
static int latent_attention_tile(const LatentArgs& a, hipStream_t stream);

static int latent_check(const LatentArgs& a, const char* who) {
  NINFER_REQUIRE(a.T > 0 && a.Hq > 0 && a.R > 0 && a.rd >= 0 && a.dim >= 0,
                 "%s: T=%d heads=%d latent=%d rotated=%d unrotated=%d", who, a.T, a.Hq, a.R, a.rd,
                 a.dim);
  NINFER_REQUIRE(a.rot_n >= 0 && a.rot_n <= a.rd && a.rot_n % 2 == 0,
                 "%s: %d turning numbers must be even and at most %d", who, a.rot_n, a.rd);
  NINFER_REQUIRE(a.rot_n == 0 || a.freq, "%s: a rotation without a table", who);
  NINFER_REQUIRE(a.page_size > 0 && a.bt_stride > 0, "%s: bad page size %d or table width %d", who,
                 a.page_size, a.bt_stride);
  NINFER_REQUIRE(a.dtype == kF32 || a.dtype == kBF16, "%s: unknown dtype %d", who, a.dtype);
  NINFER_REQUIRE(a.window >= 0, "%s: window %d must be >= 0", who, a.window);
  return 0;
}

}  // namespace ninfer

using namespace ninfer;

extern "C" int ninfer_latent_kv_write(const LatentArgs* a, hipStream_t stream) {
  if (int rc = latent_check(*a, "latent_kv_write")) return rc;
  NINFER_REQUIRE(a->dkv_stride >= a->R + a->rd, "latent_kv_write: row stride %d < %d",
                 a->dkv_stride, a->R + a->rd);
  NINFER_REQUIRE(a->eps >= 0.f, "latent_kv_write: eps must be >= 0");
  const size_t lds = (size_t)(a->rot_n > 0 ? a->rot_n : 1) * sizeof(float);
  if (a->dtype == kF32)
    latent_kv_write_kernel<float><<<a->T, 256, lds, stream>>>(*a);
  else
    latent_kv_write_kernel<bf16><<<a->T, 256, lds, stream>>>(*a);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_latent_attention(const LatentArgs* a, hipStream_t stream) {
  if (int rc = latent_check(*a, "latent_attention")) return rc;
  NINFER_REQUIRE(a->R <= 64 * kLatentMaxPerLane, "latent_attention: latent size %d exceeds %d",
                 a->R, 64 * kLatentMaxPerLane);
  NINFER_REQUIRE(a->scale > 0.f, "latent_attention: scale %g must be positive", (double)a->scale);
  if (latent_tile_takes(*a)) return latent_attention_tile(*a, stream);
  const dim3 grid(a->T, a->Hq);
  const size_t lds = (size_t)(a->R + a->rd + 64) * sizeof(float) + 64 * sizeof(int64_t);
  NINFER_REQUIRE(lds <= 64 * 1024, "latent_attention: a query of %d numbers does not fit",
                 a->R + a->rd);
  if (a->dtype == kF32)
    latent_attention_kernel<float><<<grid, 64, lds, stream>>>(*a);
  else
    latent_attention_kernel<bf16><<<grid, 64, lds, stream>>>(*a);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// ---- the matrix-core kernel ------------------------------------------------------------------
namespace ninfer {

typedef __bf16 lat_bf16x8 __attribute__((ext_vector_type(8)));
typedef float lat_f32x16 __attribute__((ext_vector_type(16)));

constexpr int kLatRows = 32;      // (token, head) rows per block
constexpr int kLatKeys = 64;      // keys per tile
constexpr int kLatColTiles = 4;   // 32-column tiles of the output per wave: latent sizes up to 512
constexpr int kLatPieces = 20;    // 16-byte pieces of a tile per thread: cached rows of up to 640 numbers

struct LatentTilePlan {
  int tiles;        // upper bound of row tiles over all requests
  int n_chunks;     // key chunks per row tile
  int chunk;        // keys per chunk (a multiple of 64)
  int dkp;          // row length of Q in LDS (numbers)
  int kstr;         // row length of a key in LDS (numbers)
  int page_shift;
  size_t lds;
};

static bool latent_tile_takes(const LatentArgs& a) {
  const int Dk = a.R + a.rd;
  return a.dtype == kBF16 && !a.force_plain && Dk % 8 == 0 && a.R <= 32 * 4 * kLatColTiles &&
         kLatKeys * (Dk / 8) <= 256 * kLatPieces &&
         (a.page_size & (a.page_size - 1)) == 0 && a.seq_row_start && a.seq_pos0 && a.S > 0 &&
         ((uintptr_t)a.pool % 16 == 0) && ((uintptr_t)a.q_abs % 16 == 0);
}

static LatentTilePlan latent_tile_plan(const LatentArgs& a) {
  LatentTilePlan p;
  const int Dk = a.R + a.rd;
  const int dk16 = (Dk + 15) / 16 * 16;
  const int cols = (a.R + 31) / 32 * 32;
  p.dkp = dk16 + 8;
  p.kstr = (dk16 > cols ? dk16 : cols) + 8;
  // row tiles: in a decode-only step every request has the same number; otherwise a bound
  // (a request's last tile may be partial; tiles that do not exist exit at once)
  p.tiles = a.max_qlen == 1 ? a.S * ((a.Hq + kLatRows - 1) / kLatRows)
                            : (int)(((int64_t)a.T * a.Hq + kLatRows - 1) / kLatRows) + a.S;
  const int key_tiles = (a.max_kv_len + kLatKeys - 1) / kLatKeys;
  // a block fills a CU (its LDS and registers): one block per CU, each with as long a walk as
  // that allows, since a block's start (Q', its first tile) costs as much as two tiles
  int want = device_cu_count() / p.tiles;
  if (want > key_tiles) want = key_tiles;
  if (want < 1) want = 1;
  const int tiles_per_chunk = (key_tiles + want - 1) / want;
  p.chunk = tiles_per_chunk * kLatKeys;
  p.n_chunks = (key_tiles + tiles_per_chunk - 1) / tiles_per_chunk;
  p.page_shift = 0;
  while ((1 << p.page_shift) < a.page_size) ++p.page_shift;
  p.lds = (size_t)kLatRows * p.dkp * 2 + (size_t)kLatKeys * p.kstr * 2 +
          2 * kLatRows * kLatKeys * 4 + kLatRows * (kLatKeys + 8) * 2 + 3 * kLatRows * 4;
  return p;
}

static int64_t latent_tile_workspace_floats(const LatentArgs& a, const LatentTilePlan& p) {
  return p.n_chunks > 1 ? (int64_t)a.T * a.Hq * p.n_chunks * (a.R + 2) : 0;
}

__global__ __launch_bounds__(256) void latent_attention_tile_kernel(LatentArgs a, LatentTilePlan pl) {
  extern __shared__ float smem[];
  const int Dk = a.R + a.rd, R = a.R, H = a.Hq;
  __bf16* Qs = (__bf16*)smem;                                   // [32][dkp]
  __bf16* Ks = Qs + kLatRows * pl.dkp;                          // [64][kstr]
  float* Sp = (float*)(Ks + kLatKeys * pl.kstr);                // [2][32][64]
  __bf16* Ps = (__bf16*)(Sp + 2 * kLatRows * kLatKeys);         // [32][72]
  float* alpha_s = (float*)(Ps + kLatRows * (kLatKeys + 8));    // [32], then m [32], l [32]
  float* m_s = alpha_s + kLatRows;
  float* l_s = m_s + kLatRows;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int lr = lane & 31, lk = lane >> 5;

  // Which request and which of its row tiles is this block's? The tiles are dealt out from
  // the last one backwards: within a request the later tiles see more keys and run longer,
  // and the long ones should start first.
  int s = -1, lt = 0;
  {
    int total = 0;
    for (int i = 0; i < a.S; ++i)
      total += ((a.seq_row_start[i + 1] - a.seq_row_start[i]) * H + kLatRows - 1) / kLatRows;
    int left = total - 1 - (int)blockIdx.x;
    for (int i = 0; i < a.S && left >= 0; ++i) {
      const int n = (a.seq_row_start[i + 1] - a.seq_row_start[i]) * H;
      const int nt = (n + kLatRows - 1) / kLatRows;
      if (left < nt) {
        s = i;
        lt = left;
        break;
      }
      left -= nt;
    }
  }
  if (s < 0) return;
  const int chunk_id = blockIdx.y;
  const int row0 = a.seq_row_start[s];
  const int n_flat = (a.seq_row_start[s + 1] - row0) * H;
  const int pos0 = a.seq_pos0[s];
  const int f0 = lt * kLatRows;                          // first flattened row of the tile
  const int rows_here = min(kLatRows, n_flat - f0);
  const int tok_first = f0 / H, tok_last = (f0 + rows_here - 1) / H;
  const int pos_last = pos0 + tok_last;
  const int lo_first = a.window > 0 ? max(0, pos0 + tok_first - a.window + 1) : 0;
  // this block's keys: its chunk of the context, cut to what its rows can see
  const int k_begin = max(chunk_id * pl.chunk, lo_first / kLatKeys * kLatKeys);
  const int k_end = min((chunk_id + 1) * pl.chunk, pos_last + 1);
  const int* bt = a.block_table + (int64_t)s * a.bt_stride;
  const __bf16* pool = (const __bf16*)a.pool;

  // Q' of the tile's rows as bfloat16, zeros in rows and columns that are not there: eight
  // threads per row
  {
    const int i = tid >> 3;
    const float* src = nullptr;
    if (i < rows_here) {
      const int f = f0 + i;
      src = a.q_abs + ((int64_t)(row0 + f / H) * H + f % H) * Dk;
    }
    // (the row has a multiple of 8 numbers and so has its place in LDS: four at a time, and
    // several loads under way)
#pragma unroll 5
    for (int d = 4 * (tid & 7); d < pl.dkp; d += 32) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (src && d < Dk) v = *(const float4*)(src + d);
      __bf16* dst = Qs + i * pl.dkp + d;
      dst[0] = (__bf16)v.x;
      dst[1] = (__bf16)v.y;
      dst[2] = (__bf16)v.z;
      dst[3] = (__bf16)v.w;
    }
  }
  {   // the columns of a key's row beyond its numbers are read as zeros and never written again
    const int pad = pl.kstr - Dk;
    for (int e = tid; e < kLatKeys * pad; e += 256) Ks[(e / pad) * pl.kstr + Dk + e % pad] = (__bf16)0.f;
  }
  __syncthreads();

  // softmax threads: row tid / 8, keys 8 (tid % 8) .. + 7 of a tile
  const int sm_row = tid >> 3, sm_part = tid & 7;
  int sm_pos = -1, sm_lo = 0;
  if (sm_row < rows_here) {
    sm_pos = pos0 + (f0 + sm_row) / H;
    sm_lo = a.window > 0 ? max(0, sm_pos - a.window + 1) : 0;
  }
  float m_run = -INFINITY, l_run = 0.f;

  lat_f32x16 acc[kLatColTiles];
#pragma unroll
  for (int c = 0; c < kLatColTiles; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
  const int n_ct = (R + 31) / 32;
  const int ct_per_wave = (n_ct + 3) / 4;
  const int ksteps = (Dk + 15) / 16;
  const int ks_half = (ksteps + 1) / 2;
  const int cpr = Dk / 8;   // 16-byte pieces of a cached row

  // A tile's keys travel page -> registers -> LDS; the loads of the next tile are issued before
  // the products of this one, so that their way from memory is hidden behind them.
  lat_bf16x8 next[kLatPieces];
  int piece[kLatPieces];   // key of the tile << 16 | first number of the piece; -1: none
#pragma unroll
  for (int i = 0; i < kLatPieces; ++i) {
    const int e = tid + 256 * i;
    piece[i] = e < kLatKeys * cpr ? ((e / cpr) << 16) | (8 * (e % cpr)) : -1;
  }
  auto fetch = [&](int kt) {
#pragma unroll
    for (int i = 0; i < kLatPieces; ++i) {
      lat_bf16x8 v;
#pragma unroll
      for (int x = 0; x < 8; ++x) v[x] = (__bf16)0.f;
      if (piece[i] >= 0) {
        const int kp = kt + (piece[i] >> 16);
        if (kp <= pos_last) {
          const int page = bt[kp >> pl.page_shift];
          if (page >= 0)
            v = *(const lat_bf16x8*)(pool + ((int64_t)page * a.page_size + (kp & (a.page_size - 1))) * Dk +
                                     (piece[i] & 0xffff));
        }
      }
      next[i] = v;
    }
  };
  if (k_begin < k_end) fetch(k_begin);
  for (int kt = k_begin; kt < k_end; kt += kLatKeys) {
    // 1. the tile's keys into LDS as they lie in their pages
#pragma unroll
    for (int i = 0; i < kLatPieces; ++i)
      if (piece[i] >= 0)
        *(lat_bf16x8*)(Ks + (piece[i] >> 16) * pl.kstr + (piece[i] & 0xffff)) = next[i];
    if (kt + kLatKeys < k_end) fetch(kt + kLatKeys);
    lds_barrier();   // (orders LDS traffic only: the next tile's loads stay under way)
    // 2. S = Q' K^T: wave w meets keys 32 (w & 1) .. + 31 over one half of the numbers
    {
      const int n = w & 1, kh = w >> 1;
      lat_f32x16 sacc;
#pragma unroll
      for (int i = 0; i < 16; ++i) sacc[i] = 0.f;
      const int s_lo = kh ? ks_half : 0, s_hi = kh ? ksteps : ks_half;
      const __bf16* qrow = Qs + lr * pl.dkp + 8 * lk;
      const __bf16* krow = Ks + (32 * n + lr) * pl.kstr + 8 * lk;
      int st = s_lo;
      for (; st + 6 <= s_hi; st += 6) {   // six steps' operands are read before the first product
        lat_bf16x8 qf[6], kf[6];
#pragma unroll
        for (int u = 0; u < 6; ++u) {
          qf[u] = *(const lat_bf16x8*)(qrow + 16 * (st + u));
          kf[u] = *(const lat_bf16x8*)(krow + 16 * (st + u));
        }
#pragma unroll
        for (int u = 0; u < 6; ++u) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[u], kf[u], sacc, 0, 0, 0);
      }
      for (; st < s_hi; ++st) {
        const lat_bf16x8 qf = *(const lat_bf16x8*)(qrow + 16 * st);
        const lat_bf16x8 kf = *(const lat_bf16x8*)(krow + 16 * st);
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf, kf, sacc, 0, 0, 0);
      }
      // the lane holds key 32 n + lr for rows 8 q + 4 lk + r in register 4 q + r
      float* sp = Sp + kh * kLatRows * kLatKeys + 32 * n + lr;
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 4; ++r) sp[(8 * q + 4 * lk + r) * kLatKeys] = sacc[4 * q + r];
    }
    lds_barrier();   // (orders LDS traffic only: the next tile's loads stay under way)
    // 3. softmax of the tile, 32-bit: eight lanes per row
    {
      float sv[8];
      float mx = -INFINITY;
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const int j = 8 * sm_part + x;
        const int kp = kt + j;
        const float v = (Sp[sm_row * kLatKeys + j] + Sp[kLatRows * kLatKeys + sm_row * kLatKeys + j]) * a.scale;
        const bool see = kp <= sm_pos && kp >= sm_lo;
        sv[x] = see ? v : -INFINITY;
        mx = fmaxf(mx, sv[x]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
      const float m_new = fmaxf(m_run, mx);
      float al = 1.f, sum = 0.f;
      lat_bf16x8 pv;
      if (m_new == -INFINITY) {   // nothing seen so far
#pragma unroll
        for (int x = 0; x < 8; ++x) pv[x] = (__bf16)0.f;
      } else {
        al = expf(m_run - m_new);   // 0 while m_run is minus infinity
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          const float p = expf(sv[x] - m_new);
          pv[x] = (__bf16)p;
          sum += p;
        }
      }
      sum += __shfl_xor(sum, 1, 64);
      sum += __shfl_xor(sum, 2, 64);
      sum += __shfl_xor(sum, 4, 64);
      l_run = l_run * al + sum;
      m_run = m_new;
      *(lat_bf16x8*)(Ps + sm_row * (kLatKeys + 8) + 8 * sm_part) = pv;
      if (sm_part == 0) alpha_s[sm_row] = al;
    }
    lds_barrier();   // (orders LDS traffic only: the next tile's loads stay under way)
    // 4. O = O alpha + P V on this wave's column tiles
    {
      const float al = alpha_s[lr];   // every register of the lane belongs to row lr
      lat_bf16x8 pf[4];
#pragma unroll
      for (int st = 0; st < 4; ++st)
        pf[st] = *(const lat_bf16x8*)(Ps + lr * (kLatKeys + 8) + 16 * st + 8 * lk);
#pragma unroll
      for (int c = 0; c < kLatColTiles; ++c) {
        const int ct = w * ct_per_wave + c;
        if (c < ct_per_wave && ct < n_ct) {
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[c][i] *= al;
          const __bf16* vcol = Ks + 32 * ct + lr;
#pragma unroll
          for (int st = 0; st < 4; ++st) {
            lat_bf16x8 vf;
#pragma unroll
            for (int x = 0; x < 8; ++x) vf[x] = vcol[(16 * st + 8 * lk + x) * pl.kstr];
            // A = V^T: lane holds column 32 ct + lr for 8 keys; B = P^T: row lr for the same keys
            acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[st], acc[c], 0, 0, 0);
          }
        }
      }
    }
    lds_barrier();   // (orders LDS traffic only: the next tile's loads stay under way)
  }

  if (sm_part == 0) {
    m_s[sm_row] = m_run;
    l_s[sm_row] = l_run;
  }
  __syncthreads();
  // With A = V^T and B = P^T the lane holds row lr of the tile (a (token, head) pair) and the
  // columns 32 ct + 8 q + 4 lk + r in register 4 q + r.
  if (lr < rows_here) {
    const int f = f0 + lr;
    const int t = row0 + f / H, h = f % H;
    const float l = l_s[lr], m = m_s[lr];
    if (pl.n_chunks == 1) {
      float inv = l > 0.f ? 1.f / l : 0.f;
      if (a.gate) {
        const float g = __bfloat162float(((const bf16*)a.gate)[(int64_t)t * a.gate_stride + h]);
        inv *= 1.f / (1.f + expf(-g));
      }
      __bf16* orow = (__bf16*)a.out + ((int64_t)t * H + h) * R;
#pragma unroll
      for (int c = 0; c < kLatColTiles; ++c) {
        const int ct = w * ct_per_wave + c;
        if (c < ct_per_wave && ct < n_ct) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int d = 32 * ct + 8 * q + 4 * lk + r;
              if (d < R) orow[d] = (__bf16)(acc[c][4 * q + r] * inv);
            }
        }
      }
    } else {
      float* part = a.workspace + (((int64_t)t * H + h) * pl.n_chunks + chunk_id) * (R + 2);
      if (w == 0 && lk == 0) {
        part[R] = m;
        part[R + 1] = l;
      }
#pragma unroll
      for (int c = 0; c < kLatColTiles; ++c) {
        const int ct = w * ct_per_wave + c;
        if (c < ct_per_wave && ct < n_ct) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int d = 32 * ct + 8 * q + 4 * lk + r;
              if (d < R) part[d] = acc[c][4 * q + r];
            }
        }
      }
    }
  }
}

// out[t, h] = sum_c e^(m_c - M) O_c / sum_c e^(m_c - M) l_c over the chunks that saw keys.
__global__ void latent_attention_merge_kernel(LatentArgs a, int n_chunks) {
  extern __shared__ float smem[];   // [n_chunks] weight of each chunk: e^(m_c - M) / L (0: saw no key)
  __shared__ float red[16];
  const int64_t th = blockIdx.x;
  const int R = a.R;
  const float* part = a.workspace + th * n_chunks * (R + 2);
  float M = -INFINITY;
#pragma unroll 8
  for (int c = 0; c < n_chunks; ++c) M = fmaxf(M, part[c * (R + 2) + R]);
  float mine = 0.f;
  for (int c = threadIdx.x; c < n_chunks; c += blockDim.x) {
    const float m = part[c * (R + 2) + R];
    const float wgt = m > -INFINITY ? expf(m - M) : 0.f;
    smem[c] = wgt;
    mine += wgt * part[c * (R + 2) + R + 1];
  }
  const float L = block_sum(mine, red);   // (its barriers publish the weights)
  float inv = L > 0.f ? 1.f / L : 0.f;
  if (a.gate) {
    const int t = (int)(th / a.Hq), h = (int)(th % a.Hq);
    const float g = __bfloat162float(((const bf16*)a.gate)[(int64_t)t * a.gate_stride + h]);
    inv *= 1.f / (1.f + expf(-g));
  }
  __bf16* orow = (__bf16*)a.out + th * R;
  for (int d = threadIdx.x; d < R; d += blockDim.x) {
    // (a chunk that saw no key left zeros and has weight 0: no branch, so that the loads of
    // several chunks are under way together)
    float o = 0.f;
#pragma unroll 8
    for (int c = 0; c < n_chunks; ++c) o = fmaf(smem[c], part[c * (R + 2) + d], o);
    orow[d] = (__bf16)(o * inv);
  }
}

static int latent_attention_tile(const LatentArgs& a, hipStream_t stream) {
  const LatentTilePlan p = latent_tile_plan(a);
  NINFER_REQUIRE(p.lds <= 160 * 1024, "latent_attention: rows of %d numbers do not fit the LDS",
                 a.R + a.rd);
  const int64_t need = latent_tile_workspace_floats(a, p);
  NINFER_REQUIRE(need == 0 || (a.workspace && a.workspace_floats >= need),
                 "latent_attention: the workspace holds %lld floats, %lld are needed",
                 (long long)a.workspace_floats, (long long)need);
  auto kern = latent_attention_tile_kernel;
  if (p.lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)p.lds);
    if (e != hipSuccess) return set_error(-2, "latent_attention: cannot get %zu bytes of LDS", p.lds);
  }
  kern<<<dim3(p.tiles, p.n_chunks), 256, p.lds, stream>>>(a, p);
  NINFER_LAUNCH_CHECK();
  if (p.n_chunks > 1) {
    const int block = a.R >= 256 ? 256 : (a.R + 63) / 64 * 64;
    latent_attention_merge_kernel<<<(unsigned)((int64_t)a.T * a.Hq), block, p.n_chunks * sizeof(float), stream>>>(a, p.n_chunks);
    NINFER_LAUNCH_CHECK();
  }
  return 0;
}

}  // namespace ninfer

// 32-bit floats of workspace that a step of this shape needs (0: none).
extern "C" long long ninfer_latent_attention_workspace_floats(const ninfer::LatentArgs* a) {
  if (!ninfer::latent_tile_takes(*a)) return 0;
  return ninfer::latent_tile_workspace_floats(*a, ninfer::latent_tile_plan(*a));
}
