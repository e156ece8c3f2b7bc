// Softmax attention over the paged cache on the matrix cores (bf16 rows and cache) for keys of
// D and values of Dv numbers (any multiples of 8 up to 128 each), with a window or none and with
// a sink or none. The sizes the 64/128 kernels of attention_prefill.hip do not take run here.
//
// Prompt portions: a block of four waves owns one kv head and a tile of rows of one request; a
// wave owns 32 rows of one query head (HB = 4, 2 or 1 query heads of the kv head side by side,
// 4 / HB groups of 32 rows), so that all waves meet the same keys and values. These are walked
// in tiles of 64 keys aligned to absolute positions, from the tile that holds the first key the
// tile's first row sees (its position - window + 1, or 0): global memory -> registers (one tile
// ahead) -> LDS, two buffers, one barrier per tile. A key row lies in LDS padded with zeros to
// DP = 16 KS numbers, a value row to VP = 32 DB. With v_mfma_f32_32x32x16_bf16 a wave computes
//   S^T[key][row] = K Q^T         (A = key rows from LDS, B = the queries in registers)
// whose accumulators give lane l the scores of row l % 32 for keys 8 (v / 4) + 4 (l / 32) +
// v % 4 of each block of 32 keys; scale, mask and the online softmax run on them in 32-bit (the
// two lanes of a row meet by one cross-lane step); the probabilities, rounded to bf16 in place,
// are the B operand of
//   O^T[value column][row] += V^T P^T   (A = V^T: the transposing LDS read hands a lane four
//                                        consecutive keys of one value column)
// with the contraction index numbered as the lanes hold it. A sink is a key with score 0 and
// no value: the running maximum starts at 0 and the running sum at 1.
//
// Single rows (decode steps): a block of two waves owns one row and one kv head, the query heads
// of the kv head (at most 32) are the tile's rows, so that the keys and values of the kv head
// are read once for all of them; wave w takes keys 32 w .. + 31 of every tile with a running
// maximum, sum and output of its own, and the two meet through LDS at the end. When rows and
// kv heads alone do not fill the GPU, a row's visible keys are cut into chunks of whole tiles
// over several blocks, whose records a second kernel merges.
//
// No load stands under a condition: a key that is not there (beyond the last row's position,
// or before the first key any row of the tile sees, whose page a window may have given back)
// loads the nearest key that is there in its place; it is masked, and what it holds is finite.
#include "attention.h"

namespace ninfer {

typedef __bf16 at_bf16x8 __attribute__((ext_vector_type(8)));
typedef float at_f32x16 __attribute__((ext_vector_type(16)));
typedef short at_short4 __attribute__((ext_vector_type(4)));
typedef short at_short8 __attribute__((ext_vector_type(8)));
typedef unsigned int at_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) at_short4 at_lds_short4;

constexpr float kAtLog2e = 1.44269504088896f;

// What both kernels share: the pieces of a tile that a thread moves, and the products of one
// wave with 32 keys of a tile.
template <int KS, int DB, int NT>
struct TileMover {
  static constexpr int DP = 16 * KS, KROW = DP + 8, VP = 32 * DB, VROW = VP + 8;
  static constexpr int TILE = 64 * KROW + 64 * VROW;   // elements of one buffer
  static constexpr int KP = (64 * 2 * KS + NT - 1) / NT, VPC = (64 * 4 * DB + NT - 1) / NT;
  int k_key[KP], k_src[KP], v_key[VPC], v_src[VPC];
  bool k_ok[KP], v_ok[VPC];
  at_u32x4 kreg[KP], vreg[VPC];

  __device__ __forceinline__ void init(int tid, int dim, int vdim) {
    const int cpk = dim / 8, cpv = vdim / 8;
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int p = i * NT + tid;
      k_ok[i] = p < 64 * cpk;
      const int pc = min(p, 64 * cpk - 1);
      k_key[i] = pc / cpk;
      k_src[i] = (pc % cpk) * 8;
    }
#pragma unroll
    for (int i = 0; i < VPC; ++i) {
      const int p = i * NT + tid;
      v_ok[i] = p < 64 * cpv;
      const int pc = min(p, 64 * cpv - 1);
      v_key[i] = pc / cpv;
      v_src[i] = (pc % cpv) * 8;
    }
  }
  // keys k0 .. k0 + 63, each clamped to [lo, hi]
  __device__ __forceinline__ void load(const unsigned short* kpool, const unsigned short* vpool,
                                       const int* bt, int ps_shift, int ps_mask, int page_size,
                                       int Hkv, int g, int dim, int vdim, int k0, int lo, int hi) {
#pragma unroll
    for (int i = 0; i < KP; ++i) {
      const int j = max(min(k0 + k_key[i], hi), lo);
      const int64_t at = ((int64_t)bt[j >> ps_shift] * Hkv + g) * page_size + (j & ps_mask);
      kreg[i] = *(const at_u32x4*)(kpool + at * dim + k_src[i]);
    }
#pragma unroll
    for (int i = 0; i < VPC; ++i) {
      const int j = max(min(k0 + v_key[i], hi), lo);
      const int64_t at = ((int64_t)bt[j >> ps_shift] * Hkv + g) * page_size + (j & ps_mask);
      vreg[i] = *(const at_u32x4*)(vpool + at * vdim + v_src[i]);
    }
  }
  __device__ __forceinline__ void store(unsigned short* ks) const {
    unsigned short* vs = ks + 64 * KROW;
#pragma unroll
    for (int i = 0; i < KP; ++i)
      if (k_ok[i]) *(at_u32x4*)(ks + k_key[i] * KROW + k_src[i]) = kreg[i];
#pragma unroll
    for (int i = 0; i < VPC; ++i)
      if (v_ok[i]) *(at_u32x4*)(vs + v_key[i] * VROW + v_src[i]) = vreg[i];
  }
};

// One wave, 32 keys (block kb of the tile at `ks_`): scores, mask, online softmax, values.
// `q_pos`: the lane's row's position; `lo_pos`: the first position it sees; `masked`: some key
// of the block may be invisible to some row.
template <int KS, int DB>
__device__ __forceinline__ void wave_keys(const unsigned short* ks_, const unsigned short* vs_,
                                          int kb, int c, int hi, int v_lane,
                                          const at_bf16x8* qf, float pre, int key0, int q_pos,
                                          int lo_pos, bool masked, float& m, float& l,
                                          at_f32x16* o) {
  constexpr int KROW = 16 * KS + 8, VROW = 32 * DB + 8;
  at_f32x16 s;
#pragma unroll
  for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const at_bf16x8 kf = *(const at_bf16x8*)(ks_ + (32 * kb + c) * KROW + 16 * ks + 8 * hi);
    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], s, 0, 0, 0);
  }
  float mx = -__builtin_inff();
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    float x = s[v] * pre;
    if (masked) {
      const int kp = key0 + 8 * (v >> 2) + 4 * hi + (v & 3);
      if (kp > q_pos || kp < lo_pos) x = -__builtin_inff();
    }
    s[v] = x;
    mx = fmaxf(mx, x);
  }
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  const float m_new = fmaxf(m, mx);
  if (__any(m_new > m)) {
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    l *= alpha;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[db][v] *= alpha;
    m = m_new;
  }
  at_bf16x8 pf[2];
  float psum = 0.f;
#pragma unroll
  for (int hh = 0; hh < 2; ++hh)
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) {
      const float p = __builtin_amdgcn_exp2f(s[8 * hh + jj] - m);
      psum += p;
      pf[hh][jj] = (__bf16)p;
    }
  l += psum + __shfl_xor(psum, 32, 64);
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const unsigned short* p = vs_ + v_lane + (32 * kb + 16 * hh) * VROW + 32 * db;
      const at_short4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((at_lds_short4*)p);
      const at_short4 up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((at_lds_short4*)(p + 8 * VROW));
      at_short8 both;
      both.s0 = lo.x; both.s1 = lo.y; both.s2 = lo.z; both.s3 = lo.w;
      both.s4 = up.x; both.s5 = up.y; both.s6 = up.z; both.s7 = up.w;
      o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(at_bf16x8, both), pf[hh],
                                                      o[db], 0, 0, 0);
    }
}

template <int KS, int DB>
__global__ __launch_bounds__(256, 2) void attention_tiles_kernel(AttnArgs a, int HB, int first_seq) {
  using Mover = TileMover<KS, DB, 256>;
  constexpr int KROW = Mover::KROW, VROW = Mover::VROW, TILE = Mover::TILE;
  extern __shared__ __attribute__((aligned(16))) unsigned short lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, hi = lane >> 5;
  const int hpg = a.Hq / a.Hkv;
  const int RT = 32 * (4 / HB);
  const int g = blockIdx.y / (hpg / HB);
  const int h = g * hpg + (blockIdx.y % (hpg / HB)) * HB + wave % HB;
  const int rs = wave / HB;

  // which request and which of its row tiles
  int seq = -1, row0 = 0, n_rows = 0;
  {
    int idx = gridDim.x - 1 - blockIdx.x;   // the last row tiles of a request walk the most keys: first
    for (int s = first_seq; s < a.S; ++s) {
      const int b = a.seq_row_start[s], e = a.seq_row_start[s + 1];
      const int nt = (e - b + RT - 1) / RT;
      if (idx < nt) {
        seq = s;
        row0 = b + idx * RT;
        n_rows = min(RT, e - row0);
        break;
      }
      idx -= nt;
    }
  }
  if (seq < 0) return;
  const int pos_first = a.positions[row0], pos_last = pos_first + n_rows - 1;
  const int key_lo = a.window > 0 ? max(0, pos_first - a.window + 1) : 0;   // the first key any row sees
  const int* bt = a.block_table + (int64_t)seq * a.bt_stride;
  const int ps_shift = __builtin_ctz(a.page_size), ps_mask = a.page_size - 1;
  const int dim = a.D, vdim = a.Dv;
  const unsigned short* kpool = (const unsigned short*)a.kpool;
  const unsigned short* vpool = (const unsigned short*)a.vpool;

  // zeros everywhere once: the padding columns stay zero, the rest is overwritten
  for (int i = tid; i < 2 * TILE / 8; i += 256) ((at_u32x4*)lds)[i] = at_u32x4{0u, 0u, 0u, 0u};

  Mover mv;
  mv.init(tid, dim, vdim);

  // this lane's queries (B operand): row c of the wave, dims 16 ks + 8 hi .. + 7
  const bool wave_live = rs * 32 < n_rows;
  const int q_local = rs * 32 + c;
  const bool q_valid = q_local < n_rows;
  const int q_pos = pos_first + q_local;
  const int lo_pos = a.window > 0 ? q_pos - a.window + 1 : 0;
  const int wave_first = pos_first + rs * 32;
  const int wave_last = pos_first + min(rs * 32 + 31, n_rows - 1);
  const int wave_lo = a.window > 0 ? wave_first - a.window + 1 : 0;
  at_bf16x8 qf[KS];
  {
    const unsigned short* qr = (const unsigned short*)a.q +
                               (int64_t)(row0 + (q_valid ? q_local : 0)) * a.q_stride + h * dim;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 16 * ks + 8 * hi;
      at_u32x4 v = {0u, 0u, 0u, 0u};
      if (d < dim) v = *(const at_u32x4*)(qr + d);
      qf[ks] = __builtin_bit_cast(at_bf16x8, v);
    }
  }
  const float pre = a.scale * kAtLog2e;   // scores in units of log 2

  at_f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  float m = a.sink ? 0.f : -1e30f, l = a.sink ? 1.f : 0.f;

  // the transposing read's address of this lane inside a value tile: lane s of a group of 16
  // fetches key s / 4 (+ 4 hi), value columns 16 (group % 2) + 4 (s % 4) .. + 3
  const int s16 = lane & 15, q4 = lane >> 4;
  const int v_lane = (4 * hi + s16 / 4) * VROW + 16 * (q4 & 1) + 4 * (s16 & 3);

  const int kt0 = key_lo / 64, n_kt = pos_last / 64 + 1;
  mv.load(kpool, vpool, bt, ps_shift, ps_mask, a.page_size, a.Hkv, g, dim, vdim, kt0 * 64, key_lo,
          pos_last);
  __syncthreads();   // the zeros are written
  for (int kt = kt0; kt < n_kt; ++kt) {
    const int k0 = kt * 64, buf = (kt - kt0) & 1;
    mv.store(lds + buf * TILE);
    __syncthreads();
    if (kt + 1 < n_kt)
      mv.load(kpool, vpool, bt, ps_shift, ps_mask, a.page_size, a.Hkv, g, dim, vdim, k0 + 64, key_lo,
              pos_last);
    if (!wave_live || k0 > wave_last || k0 + 63 < wave_lo) continue;
    const unsigned short* ks_ = lds + buf * TILE;
    const unsigned short* vs_ = ks_ + 64 * KROW;
    // some row of the wave does not see every key of the tile
    const bool masked = k0 + 63 > wave_first || (a.window > 0 && k0 < wave_last - a.window + 1);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
      wave_keys<KS, DB>(ks_, vs_, kb, c, hi, v_lane, qf, pre, k0 + 32 * kb, q_pos, lo_pos, masked,
                        m, l, o);
  }
  if (!q_valid) return;
  // lane holds, for row c, value columns 32 db + 8 (v / 4) + 4 hi + v % 4
  const float r = 1.f / l;
  unsigned short* orow = (unsigned short*)a.out + ((int64_t)(row0 + q_local) * a.Hq + h) * vdim;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int col = 32 * db + 8 * v4 + 4 * hi;
      if (col < vdim) {   // value sizes are multiples of 8: four columns are there together
        union { __bf16 b[4]; uint2 u; } w;
#pragma unroll
        for (int e = 0; e < 4; ++e) w.b[e] = (__bf16)(o[db][4 * v4 + e] * r);
        *(uint2*)(orow + col) = w.u;
      }
    }
}

// `tiles_per_chunk`, `n_chunks`: the visible keys of a row are cut into chunks of so many tiles
// (counted from the tile that holds the row's first visible key), one block each
// (blockIdx.z), when rows and kv heads alone do not fill the GPU; every block then leaves a
// record {m, l, o[Dv]} per head (m in units of log 2) that the merge kernel puts together.
template <int KS, int DB>
__global__ __launch_bounds__(128, 2) void attention_tiles_heads_kernel(AttnArgs a, int tiles_per_chunk,
                                                                    int n_chunks) {
  using Mover = TileMover<KS, DB, 128>;
  constexpr int KROW = Mover::KROW, VROW = Mover::VROW, TILE = Mover::TILE;
  extern __shared__ __attribute__((aligned(16))) unsigned short lds[];

  const int tid = threadIdx.x, lane = tid & 63, kb = tid >> 6;
  const int c = lane & 31, hi = lane >> 5;
  const int hpg = a.Hq / a.Hkv;
  const int t = blockIdx.x, g = blockIdx.y, ch = blockIdx.z;
  const int pos = a.positions[t];
  const int first = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int dim = a.D, vdim = a.Dv;
  const bool q_valid = c < hpg;
  const int h = g * hpg + (q_valid ? c : 0);
  const int kt0 = first / 64 + ch * tiles_per_chunk;
  const int n_kt = min(pos / 64 + 1, kt0 + tiles_per_chunk);
  float* rec = n_chunks > 1 ? a.workspace + (((int64_t)t * a.Hq + h) * n_chunks + ch) * (2 + vdim) : nullptr;
  if (kt0 >= n_kt) {   // nothing of this chunk is visible: a record that counts for nothing
    if (q_valid && kb == 0) {
      if (hi == 0) {
        rec[0] = -1e30f;
        rec[1] = 0.f;
      }
      for (int col = 4 * hi; col < vdim; col += 8) {   // (a record starts at an even float: 8-byte stores)
        *(float2*)(rec + 2 + col) = make_float2(0.f, 0.f);
        *(float2*)(rec + 4 + col) = make_float2(0.f, 0.f);
      }
    }
    return;
  }
  const int* bt = a.block_table + (int64_t)a.row_seq[t] * a.bt_stride;
  const int ps_shift = __builtin_ctz(a.page_size), ps_mask = a.page_size - 1;
  const unsigned short* kpool = (const unsigned short*)a.kpool;
  const unsigned short* vpool = (const unsigned short*)a.vpool;

  for (int i = tid; i < TILE / 8; i += 128) ((at_u32x4*)lds)[i] = at_u32x4{0u, 0u, 0u, 0u};
  Mover mv;
  mv.init(tid, dim, vdim);

  at_bf16x8 qf[KS];
  {
    const unsigned short* qr = (const unsigned short*)a.q + (int64_t)t * a.q_stride + h * dim;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 16 * ks + 8 * hi;
      at_u32x4 v = {0u, 0u, 0u, 0u};
      if (d < dim) v = *(const at_u32x4*)(qr + d);
      qf[ks] = __builtin_bit_cast(at_bf16x8, v);
    }
  }
  const float pre = a.scale * kAtLog2e;
  at_f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  // the sink counts once: in the first wave's sum of the first chunk
  const bool with_sink = a.sink && kb == 0 && ch == 0;
  float m = with_sink ? 0.f : -1e30f, l = with_sink ? 1.f : 0.f;
  const int s16 = lane & 15, q4 = lane >> 4;
  const int v_lane = (4 * hi + s16 / 4) * VROW + 16 * (q4 & 1) + 4 * (s16 & 3);

  mv.load(kpool, vpool, bt, ps_shift, ps_mask, a.page_size, a.Hkv, g, dim, vdim, kt0 * 64, first, pos);
  __syncthreads();
  for (int kt = kt0; kt < n_kt; ++kt) {
    const int k0 = kt * 64;
    if (kt > kt0) __syncthreads();   // everyone has read the tile before: it may be written over
    mv.store(lds);
    __syncthreads();
    if (kt + 1 < n_kt)
      mv.load(kpool, vpool, bt, ps_shift, ps_mask, a.page_size, a.Hkv, g, dim, vdim, k0 + 64, first, pos);
    const int key0 = k0 + 32 * kb;
    if (key0 > pos || key0 + 31 < first) continue;   // none of this wave's keys is visible
    const bool masked = key0 + 31 > pos || key0 < first;
    wave_keys<KS, DB>(lds, lds + 64 * KROW, kb, c, hi, v_lane, qf, pre, key0, pos, first, masked, m, l, o);
  }
  // the two waves meet: the second leaves its maximum, sum and output in LDS, lane by lane
  // (both hold the same rows and columns in the same places), where the tile was
  __syncthreads();
  float* x_s = (float*)lds;
  static_assert((DB * 16 + 2) * 64 * 4 <= TILE * 2, "the waves' exchange exceeds the tile's LDS");
  if (kb == 1) {
    x_s[lane] = m;
    x_s[64 + lane] = l;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) x_s[(2 + db * 16 + v) * 64 + lane] = o[db][v];
  }
  __syncthreads();
  if (kb == 1 || !q_valid) return;
  const float m2 = x_s[lane], l2 = x_s[64 + lane];
  const float mm = fmaxf(m, m2);
  const float f1 = __builtin_amdgcn_exp2f(m - mm), f2 = __builtin_amdgcn_exp2f(m2 - mm);
  if (rec) {   // one chunk of several: the record, unnormalised
    if (hi == 0) {
      rec[0] = mm;
      rec[1] = l * f1 + l2 * f2;
    }
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const int col = 32 * db + 8 * v4 + 4 * hi;
        if (col < vdim) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            rec[2 + col + e] = o[db][4 * v4 + e] * f1 + x_s[(2 + db * 16 + 4 * v4 + e) * 64 + lane] * f2;
        }
      }
    return;
  }
  const float r = 1.f / (l * f1 + l2 * f2);
  unsigned short* orow = (unsigned short*)a.out + ((int64_t)t * a.Hq + h) * vdim;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int col = 32 * db + 8 * v4 + 4 * hi;
      if (col < vdim) {
        union { __bf16 b[4]; uint2 u; } w;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          w.b[e] = (__bf16)((o[db][4 * v4 + e] * f1 + x_s[(2 + db * 16 + 4 * v4 + e) * 64 + lane] * f2) * r);
        *(uint2*)(orow + col) = w.u;
      }
    }
}

// The records of a row and head put together: out = sum_c o_c 2^(m_c - m) / sum_c l_c 2^(m_c - m).
// Lane c weighs chunk c (64 chunks at a time); the outputs' loads do not wait for each other.
__global__ __launch_bounds__(64) void attention_tiles_merge_kernel(AttnArgs a, int n_chunks) {
  const int th = blockIdx.x, lane = threadIdx.x;
  const int vdim = a.Dv, stride = 2 + vdim;
  const float* rec = a.workspace + (int64_t)th * n_chunks * stride;
  float mm = -1e30f;
  for (int c = lane; c < n_chunks; c += 64) mm = fmaxf(mm, rec[c * stride]);
  mm = wave_max(mm);
  float l = 0.f, acc[2] = {0.f, 0.f};
  for (int c0 = 0; c0 < n_chunks; c0 += 64) {
    const int c = c0 + lane;
    float f = 0.f;
    if (c < n_chunks) {
      f = __builtin_amdgcn_exp2f(rec[c * stride] - mm);
      l += rec[c * stride + 1] * f;   // (a chunk with no visible key has l = 0 and o = 0)
    }
    const int cnt = min(64, n_chunks - c0);
#pragma unroll 4
    for (int j = 0; j < cnt; ++j) {
      const float fj = __shfl(f, j, 64);
      const float* r = rec + (c0 + j) * stride + 2;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int d = lane + 64 * i;
        if (d < vdim) acc[i] = fmaf(r[d], fj, acc[i]);
      }
    }
  }
  const float inv = 1.f / wave_sum(l);
  __bf16* orow = (__bf16*)a.out + (int64_t)th * vdim;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int d = lane + 64 * i;
    if (d < vdim) orow[d] = (__bf16)(acc[i] * inv);
  }
}

// Chunks of the visible keys (whole tiles) so that the launch has about four blocks a CU, at
// least two tiles a chunk.
static void heads_plan(const AttnArgs& a, int* tiles_per_chunk, int* n_chunks) {
  const int span = a.window > 0 && a.window < a.max_kv_len ? a.window : a.max_kv_len;
  const int tiles = span / 64 + 2;   // a span of keys that starts anywhere in a tile
  const int blocks = a.T * a.Hkv;
  const int want = (4 * device_cu_count() + blocks - 1) / blocks;
  int per = (tiles + want - 1) / want;
  if (per < 2) per = 2;
  int n = (tiles + per - 1) / per;
  // as many chunks as the workspace holds records for; without one, a block walks a row's
  // keys alone
  while (n > 1 && (!a.workspace || a.workspace_floats < (int64_t)a.T * a.Hq * n * (2 + a.Dv))) {
    per = a.workspace ? per + 1 : tiles;
    n = (tiles + per - 1) / per;
  }
  *tiles_per_chunk = per;
  *n_chunks = n;
}

bool attention_tiles_takes(const AttnArgs& a) {
  const int dv = a.Dv > 0 ? a.Dv : a.D;
  return a.dtype == kBF16 && a.D % 8 == 0 && dv % 8 == 0 && a.D <= 128 && dv <= 128 &&
         a.q_stride % 8 == 0 && (a.page_size & (a.page_size - 1)) == 0 && !a.slopes &&
         a.seq_row_start != nullptr;
}

bool attention_tiles_heads_takes(const AttnArgs& a) {
  return attention_tiles_takes(a) && a.Hq / a.Hkv <= 32 && a.row_seq != nullptr;
}

template <typename K>
static int raise_lds(K kern, size_t lds, bool* raised) {
  if (lds > 64 * 1024 && !*raised) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return set_error(-2, "paged_attention: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
    *raised = true;
  }
  return 0;
}

template <int KS, int DB>
static int launch_tiles(const AttnArgs& a, int first_seq, hipStream_t stream) {
  const int hpg = a.Hq / a.Hkv;
  const int HB = hpg % 4 == 0 ? 4 : hpg % 2 == 0 ? 2 : 1;
  const int RT = 32 * (4 / HB);
  const size_t lds = 2 * TileMover<KS, DB, 256>::TILE * sizeof(unsigned short);
  auto kern = attention_tiles_kernel<KS, DB>;
  static bool raised = false;   // per instantiation
  if (int rc = raise_lds(kern, lds, &raised)) return rc;
  // (requests before first_seq bring one row each: rows 0 .. first_seq - 1)
  dim3 grid((a.T - first_seq) / RT + a.S - first_seq, a.Hkv * (hpg / HB));
  kern<<<grid, 256, lds, stream>>>(a, HB, first_seq);
  NINFER_LAUNCH_CHECK();
  return 0;
}

template <int KS, int DB>
static int launch_heads(const AttnArgs& a, hipStream_t stream) {
  const size_t lds = TileMover<KS, DB, 128>::TILE * sizeof(unsigned short);
  auto kern = attention_tiles_heads_kernel<KS, DB>;
  static bool raised = false;
  if (int rc = raise_lds(kern, lds, &raised)) return rc;
  int per, n;
  heads_plan(a, &per, &n);
  kern<<<dim3(a.T, a.Hkv, n), 128, lds, stream>>>(a, per, n);
  NINFER_LAUNCH_CHECK();
  if (n > 1) {
    attention_tiles_merge_kernel<<<a.T * a.Hq, 64, 0, stream>>>(a, n);
    NINFER_LAUNCH_CHECK();
  }
  return 0;
}

#define NINFER_AT_DISPATCH(FN, ...)                                                              \
  {                                                                                              \
    const int db = (b.Dv + 31) / 32;                                                             \
    const int ks = b.D <= 32 ? 2 : b.D <= 64 ? 4 : b.D <= 96 ? 6 : 8;                            \
    switch (ks * 8 + db) {                                                                       \
      case 2 * 8 + 1: return FN<2, 1>(__VA_ARGS__);                                              \
      case 2 * 8 + 2: return FN<2, 2>(__VA_ARGS__);                                              \
      case 2 * 8 + 3: return FN<2, 3>(__VA_ARGS__);                                              \
      case 2 * 8 + 4: return FN<2, 4>(__VA_ARGS__);                                              \
      case 4 * 8 + 1: return FN<4, 1>(__VA_ARGS__);                                              \
      case 4 * 8 + 2: return FN<4, 2>(__VA_ARGS__);                                              \
      case 4 * 8 + 3: return FN<4, 3>(__VA_ARGS__);                                              \
      case 4 * 8 + 4: return FN<4, 4>(__VA_ARGS__);                                              \
      case 6 * 8 + 1: return FN<6, 1>(__VA_ARGS__);                                              \
      case 6 * 8 + 2: return FN<6, 2>(__VA_ARGS__);                                              \
      case 6 * 8 + 3: return FN<6, 3>(__VA_ARGS__);                                              \
      case 6 * 8 + 4: return FN<6, 4>(__VA_ARGS__);                                              \
      case 8 * 8 + 1: return FN<8, 1>(__VA_ARGS__);                                              \
      case 8 * 8 + 2: return FN<8, 2>(__VA_ARGS__);                                              \
      case 8 * 8 + 3: return FN<8, 3>(__VA_ARGS__);                                              \
      default: return FN<8, 4>(__VA_ARGS__);                                                     \
    }                                                                                            \
  }

int attention_tiles(const AttnArgs& a, int first_seq, hipStream_t stream) {
  AttnArgs b = a;
  if (b.Dv <= 0) b.Dv = b.D;
  NINFER_AT_DISPATCH(launch_tiles, b, first_seq, stream)
}

int attention_tiles_heads(const AttnArgs& a, hipStream_t stream) {
  AttnArgs b = a;
  if (b.Dv <= 0) b.Dv = b.D;
  NINFER_AT_DISPATCH(launch_heads, b, stream)
}

}  // namespace ninfer
