// Differential attention for prompt portions on the matrix cores (bf16 rows and cache).
//
// A block of four waves owns one kv head and a tile of rows of one request: a pair of waves
// owns 32 rows of one query head, one wave for each map (HB = 2 or 1 query heads of the kv
// head side by side, 2 / HB groups of 32 rows), so that all waves meet the same keys and
// values and a wave's registers hold one map's output only (two blocks fit a CU, and one
// wave's softmax arithmetic runs beside another's matrix products). These are walked in tiles of 64
// keys aligned to absolute positions: global memory -> registers (one tile ahead) -> LDS, two
// buffers, one barrier per tile. A key row lies in LDS as [map 1 | map 2], each padded with
// zeros to DP = 16 KS numbers; a value row padded to VP = 32 DB.
// With v_mfma_f32_32x32x16_bf16 a wave computes, for each map,
//   S^T[key][row] = K Q^T         (A = key rows from LDS, B = the map's queries in registers)
// whose accumulators give lane l the scores of row l % 32 for keys 8 (v / 4) + 4 (l / 32) +
// v % 4 of each block of 32 keys; temperature, scale, tanh cap, causal mask and the online
// softmax run on them in 32-bit (the two lanes of a row meet by one cross-lane step); the
// probabilities, rounded to bf16 in place, are the B operand of
//   O^T[value column][row] += V^T P^T   (A = V^T: the transposing LDS read hands a lane four
//                                        consecutive keys of one value column)
// with the contraction index numbered as the lanes hold it. At the end the wave of map 2
// hands lambda O2 / l2 to its partner through LDS (the tiles' buffers, lane by lane: both hold
// the same places), which forms o = O1 / l1 - lambda O2 / l2, the head's norm over its value
// columns, the factor, and stores.
// Keys that do not exist (beyond the tile's last row) load the last row's key in their place:
// they are masked, and their values must be finite since 0 x NaN is not 0.
#include "attention_diff.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v lds_short4;

constexpr float kLog2e = 1.44269504088896f;

template <int KS, int DB>
__global__ __launch_bounds__(256, 2) void diff_attention_tiles_kernel(DiffAttnArgs a, int HB,
                                                                      int first_seq) {
  constexpr int DP = 16 * KS, KROW = 2 * DP + 8, VP = 32 * DB, VROW = VP + 8;
  constexpr int TILE = 64 * KROW + 64 * VROW;   // elements of one buffer
  extern __shared__ __attribute__((aligned(16))) unsigned short lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, hi = lane >> 5;
  const int hpg = a.Hq / a.Hkv;
  const int mp = wave & 1, unit = wave >> 1;   // the wave's map; its pair's place in the block
  const int RT = 32 * (2 / HB);
  const int g = blockIdx.y / (hpg / HB);
  const int h = g * hpg + (blockIdx.y % (hpg / HB)) * HB + unit % HB;
  const int rs = unit / HB;

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
  const int* bt = a.block_table + (int64_t)seq * a.bt_stride;
  const int ps_shift = __builtin_ctz(a.page_size), ps_mask = a.page_size - 1;
  const int dim = a.dim, vdim = a.vdim, kd = 2 * dim;
  const unsigned short* kpool = (const unsigned short*)a.kpool;
  const unsigned short* vpool = (const unsigned short*)a.vpool;

  // zeros everywhere once: the padding columns stay zero, the rest is overwritten
  for (int i = tid; i < 2 * TILE / 8; i += 256) ((u32x4*)lds)[i] = u32x4{0u, 0u, 0u, 0u};

  // this thread's pieces of a tile (16 bytes each): key row, column in global memory and in
  // LDS. Every load is unconditional (a load under a condition makes the compiler wait for
  // all loads at the end of the branch): a piece that does not exist loads the tile's last
  // piece once more and is not stored.
  int k_key[KS], k_src[KS], k_dst[KS], v_key[DB], v_src[DB];
  bool k_ok[KS], v_ok[DB];
  {
    const int cpk = kd / 8, cpv = vdim / 8;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int p = i * 256 + tid;
      k_ok[i] = p < 64 * cpk;
      const int pc = min(p, 64 * cpk - 1);
      k_key[i] = pc / cpk;
      k_src[i] = (pc % cpk) * 8;
      k_dst[i] = k_key[i] * KROW + (k_src[i] < dim ? k_src[i] : DP + k_src[i] - dim);
    }
#pragma unroll
    for (int i = 0; i < DB; ++i) {
      const int p = i * 256 + tid;
      v_ok[i] = p < 64 * cpv;
      const int pc = min(p, 64 * cpv - 1);
      v_key[i] = pc / cpv;
      v_src[i] = (pc % cpv) * 8;
    }
  }
  u32x4 kreg[KS], vreg[DB];
#define NINFER_DIFF_LOAD_TILE(K0)                                                                 \
  {                                                                                               \
    _Pragma("unroll") for (int i = 0; i < KS; ++i) {                                              \
      const int j = min((K0) + k_key[i], pos_last);                                               \
      const int64_t at = ((int64_t)bt[j >> ps_shift] * a.Hkv + g) * a.page_size + (j & ps_mask);  \
      kreg[i] = *(const u32x4*)(kpool + at * kd + k_src[i]);                                      \
    }                                                                                             \
    _Pragma("unroll") for (int i = 0; i < DB; ++i) {                                              \
      const int j = min((K0) + v_key[i], pos_last);                                               \
      const int64_t at = ((int64_t)bt[j >> ps_shift] * a.Hkv + g) * a.page_size + (j & ps_mask);  \
      vreg[i] = *(const u32x4*)(vpool + at * vdim + v_src[i]);                                    \
    }                                                                                             \
  }
#define NINFER_DIFF_STORE_TILE(BUF)                                                               \
  {                                                                                               \
    unsigned short* ks = lds + (BUF) * TILE;                                                      \
    unsigned short* vs = ks + 64 * KROW;                                                          \
    _Pragma("unroll") for (int i = 0; i < KS; ++i)                                                \
      if (k_ok[i]) *(u32x4*)(ks + k_dst[i]) = kreg[i];                                            \
    _Pragma("unroll") for (int i = 0; i < DB; ++i)                                                \
      if (v_ok[i]) *(u32x4*)(vs + v_key[i] * VROW + v_src[i]) = vreg[i];                          \
  }

  // this lane's queries (B operand): row c of the wave, dims 16 ks + 8 hi .. + 7 of its map
  const bool wave_live = rs * 32 < n_rows;
  const int q_local = rs * 32 + c;
  const bool q_valid = q_local < n_rows;
  const int q_pos = pos_first + q_local;
  const int wave_last = pos_first + min(rs * 32 + 31, n_rows - 1);
  bf16x8 qf[KS];
  {
    const unsigned short* qr = (const unsigned short*)a.qkv +
                               (int64_t)(row0 + (q_valid ? q_local : 0)) * a.q_stride + h * kd + mp * dim;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 16 * ks + 8 * hi;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (d < dim) v = *(const u32x4*)(qr + d);
      qf[ks] = __builtin_bit_cast(bf16x8, v);
    }
  }
  // scores in units of log 2: (q . k) qscale, capped, times log2(e)
  const float qscale = a.scale * (a.t_coef == 0.f ? 1.f
                                  : 1.f + a.t_coef * logf((float)((q_pos + 1) / a.t_every) + 1.f));
  const bool capped = a.cap > 0.f;
  const float pre = capped ? qscale / a.cap * 2.f * kLog2e : qscale * kLog2e;
  const float cap2 = a.cap * kLog2e;

  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  float m = -1e30f, l = 0.f;

  // the transposing read's address of this lane inside a value tile: lane s of a group of 16
  // fetches key s / 4 (+ 4 hi), value columns 16 (group % 2) + 4 (s % 4) .. + 3
  const int s16 = lane & 15, q4 = lane >> 4;
  const int v_lane = (4 * hi + s16 / 4) * VROW + 16 * (q4 & 1) + 4 * (s16 & 3);

  NINFER_DIFF_LOAD_TILE(0)
  __syncthreads();   // the zeros are written
  const int n_kt = pos_last / 64 + 1;
  for (int kt = 0; kt < n_kt; ++kt) {
    const int k0 = kt * 64, buf = kt & 1;
    NINFER_DIFF_STORE_TILE(buf)
    __syncthreads();
    if (kt + 1 < n_kt) NINFER_DIFF_LOAD_TILE(k0 + 64)
    if (!wave_live || k0 > wave_last) continue;
    const unsigned short* ks_ = lds + buf * TILE;
    const unsigned short* vs_ = ks_ + 64 * KROW;
    const bool masked = k0 + 63 > pos_first + rs * 32;   // some row of the wave does not see every key
    f32x16 s[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kb][v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 kf = *(const bf16x8*)(ks_ + (32 * kb + c) * KROW + mp * DP + 16 * ks + 8 * hi);
        s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], s[kb], 0, 0, 0);
      }
    }
    float mx = -__builtin_inff();
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float x = s[kb][v] * pre;
        if (capped) {
          // cap tanh(y) = cap (1 - 2 / (e^(2y) + 1))
          const float e = __builtin_amdgcn_exp2f(x);
          x = cap2 * (1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f));
        }
        if (masked) {
          const int kp = k0 + 32 * kb + 8 * (v >> 2) + 4 * hi + (v & 3);
          if (kp > q_pos) x = -__builtin_inff();
        }
        s[kb][v] = x;
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
    bf16x8 pf[2][2];
    float psum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
          const float p = __builtin_amdgcn_exp2f(s[kb][8 * hh + jj] - m);
          psum += p;
          pf[kb][hh][jj] = (__bf16)p;
        }
    l += psum + __shfl_xor(psum, 32, 64);
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          const unsigned short* p = vs_ + v_lane + (32 * kb + 16 * hh) * VROW + 32 * db;
          const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)p);
          const short4v up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p + 8 * VROW));
          short8v both;
          both.s0 = lo.x; both.s1 = lo.y; both.s2 = lo.z; both.s3 = lo.w;
          both.s4 = up.x; both.s5 = up.y; both.s6 = up.z; both.s7 = up.w;
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pf[kb][hh], o[db], 0, 0, 0);
        }
  }
  // The pair meets: the wave of map 2 leaves lambda O2 / l2 in LDS, lane by lane (both waves
  // hold the same rows and columns in the same places), where the tiles were.
  __syncthreads();   // every wave has read its last tile
  float* x_s = (float*)lds + unit * (DB * 16 * 64);
  static_assert(2 * DB * 16 * 64 * 4 <= 2 * TILE * 2, "the pairs' exchange exceeds the tiles' LDS");
  if (mp == 1 && wave_live) {
    const float i2 = a.lambda / l;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) x_s[(db * 16 + v) * 64 + lane] = o[db][v] * i2;
  }
  __syncthreads();
  if (mp == 1 || !wave_live) return;
  // o = O1 / l1 - lambda O2 / l2; the norm over the head's value columns; the store. Lane
  // holds, for row c, value columns 32 db + 8 (v / 4) + 4 hi + v % 4.
  const float i1 = 1.f / l;
  float ss = 0.f;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float x = o[db][v] * i1 - x_s[(db * 16 + v) * 64 + lane];
      o[db][v] = x;
      ss += x * x;   // padding columns hold zeros
    }
  ss += __shfl_xor(ss, 32, 64);
  float r = a.out_scale;
  if (a.eps >= 0.f) r *= 1.f / sqrtf(ss / (float)vdim + a.eps);
  if (!q_valid) return;
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

bool diff_attention_tiles_takes(const DiffAttnArgs& a) {
  return a.dtype == kBF16 && a.dim % 8 == 0 && a.vdim % 8 == 0 && a.dim <= 128 && a.vdim <= 128 &&
         a.q_stride % 8 == 0 && (a.page_size & (a.page_size - 1)) == 0;
}

// Single rows (decode steps): the same products with the query heads of one kv head as the 32
// rows of the tile (at most 32 of them), so that a block reads the keys and values of its kv
// head once for all of them. A block owns one row, one kv head and one chunk of the context;
// its four waves share every tile of 64 keys: wave w takes map w / 2 and the tile's keys
// 32 (w % 2) .. + 31, with a running maximum, sum and output of its own. One buffer of LDS
// (two barriers a tile, the next tile on its way in registers meanwhile), so that four
// blocks fit a CU: what keeps the memory busy is the number of tiles under way. Every wave writes its
// part of a record {m1, l1, m2, l2, acc1[vdim], acc2[vdim]} (one record per chunk and half),
// and the merge kernel puts the records of a row and head together.
template <int KS, int DB>
__global__ __launch_bounds__(256, 2) void diff_attention_heads_kernel(DiffAttnArgs a, int chunk,
                                                                   int n_chunks) {
  constexpr int DP = 16 * KS, KROW = 2 * DP + 8, VP = 32 * DB, VROW = VP + 8;
  constexpr int TILE = 64 * KROW + 64 * VROW;
  extern __shared__ __attribute__((aligned(16))) unsigned short lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, hi = lane >> 5;
  const int mp = wave >> 1, kb = wave & 1;
  const int hpg = a.Hq / a.Hkv;
  const int t = blockIdx.x, g = blockIdx.y, ch = blockIdx.z;
  const int pos = a.positions[t];
  const int first = ch * chunk, last = min(pos, first + chunk - 1);
  const int dim = a.dim, vdim = a.vdim, kd = 2 * dim;
  const bool q_valid = c < hpg;
  const int h = g * hpg + (q_valid ? c : 0);
  float* part = a.workspace + (((int64_t)t * a.Hq + h) * (2 * n_chunks) + 2 * ch + kb) * (4 + 2 * vdim);
  if (first > pos) {   // nothing of this chunk is visible: records that count for nothing
    if (q_valid && hi == 0) {
      part[2 * mp] = -1e30f;
      part[2 * mp + 1] = 0.f;
    }
    return;
  }
  const int* bt = a.block_table + (int64_t)a.row_seq[t] * a.bt_stride;
  const int ps_shift = __builtin_ctz(a.page_size), ps_mask = a.page_size - 1;
  const unsigned short* kpool = (const unsigned short*)a.kpool;
  const unsigned short* vpool = (const unsigned short*)a.vpool;
  const int pos_last = last;   // (the name the tile macros use: no key beyond it is loaded)

  for (int i = tid; i < TILE / 8; i += 256) ((u32x4*)lds)[i] = u32x4{0u, 0u, 0u, 0u};

  int k_key[KS], k_src[KS], k_dst[KS], v_key[DB], v_src[DB];
  bool k_ok[KS], v_ok[DB];
  {
    const int cpk = kd / 8, cpv = vdim / 8;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int p = i * 256 + tid;
      k_ok[i] = p < 64 * cpk;
      const int pc = min(p, 64 * cpk - 1);
      k_key[i] = pc / cpk;
      k_src[i] = (pc % cpk) * 8;
      k_dst[i] = k_key[i] * KROW + (k_src[i] < dim ? k_src[i] : DP + k_src[i] - dim);
    }
#pragma unroll
    for (int i = 0; i < DB; ++i) {
      const int p = i * 256 + tid;
      v_ok[i] = p < 64 * cpv;
      const int pc = min(p, 64 * cpv - 1);
      v_key[i] = pc / cpv;
      v_src[i] = (pc % cpv) * 8;
    }
  }
  u32x4 kreg[KS], vreg[DB];

  bf16x8 qf[KS];
  {
    const unsigned short* qr = (const unsigned short*)a.qkv + (int64_t)t * a.q_stride + h * kd + mp * dim;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = 16 * ks + 8 * hi;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (d < dim) v = *(const u32x4*)(qr + d);
      qf[ks] = __builtin_bit_cast(bf16x8, v);
    }
  }
  const float qscale = a.scale * (a.t_coef == 0.f ? 1.f
                                  : 1.f + a.t_coef * logf((float)((pos + 1) / a.t_every) + 1.f));
  const bool capped = a.cap > 0.f;
  const float pre = capped ? qscale / a.cap * 2.f * kLog2e : qscale * kLog2e;
  const float cap2 = a.cap * kLog2e;

  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  float m = -1e30f, l = 0.f;
  const int s16 = lane & 15, q4 = lane >> 4;
  const int v_lane = (32 * kb + 4 * hi + s16 / 4) * VROW + 16 * (q4 & 1) + 4 * (s16 & 3);

  NINFER_DIFF_LOAD_TILE(first)
  __syncthreads();
  const int n_kt = (last - first) / 64 + 1;
  for (int kt = 0; kt < n_kt; ++kt) {
    const int k0 = first + kt * 64;
    if (kt > 0) __syncthreads();   // everyone has read the tile before: it may be written over
    NINFER_DIFF_STORE_TILE(0)
    __syncthreads();
    if (kt + 1 < n_kt) NINFER_DIFF_LOAD_TILE(k0 + 64)
    if (k0 + 32 * kb > last) continue;   // none of this wave's keys is there
    const unsigned short* ks_ = lds;
    const unsigned short* vs_ = ks_ + 64 * KROW;
    f32x16 s;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 kf = *(const bf16x8*)(ks_ + (32 * kb + c) * KROW + mp * DP + 16 * ks + 8 * hi);
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], s, 0, 0, 0);
    }
    const bool masked = k0 + 32 * kb + 31 > last;
    float mx = -__builtin_inff();
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      float x = s[v] * pre;
      if (capped) {
        const float e = __builtin_amdgcn_exp2f(x);
        x = cap2 * (1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f));
      }
      if (masked) {
        const int kp = k0 + 32 * kb + 8 * (v >> 2) + 4 * hi + (v & 3);
        if (kp > last) x = -__builtin_inff();
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
    bf16x8 pf[2];
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
        const unsigned short* p = vs_ + v_lane + 16 * hh * VROW + 32 * db;
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)p);
        const short4v up = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(p + 8 * VROW));
        short8v both;
        both.s0 = lo.x; both.s1 = lo.y; both.s2 = lo.z; both.s3 = lo.w;
        both.s4 = up.x; both.s5 = up.y; both.s6 = up.z; both.s7 = up.w;
        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pf[hh], o[db], 0, 0, 0);
      }
  }
  if (!q_valid) return;
  if (hi == 0) {
    part[2 * mp] = m * 0.6931471805599453f;   // the merge kernel counts in natural logarithms
    part[2 * mp + 1] = l;
  }
  float* acc = part + 4 + mp * vdim;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int col = 32 * db + 8 * v4 + 4 * hi;
      if (col < vdim)
        *(float4*)(acc + col) = make_float4(o[db][4 * v4], o[db][4 * v4 + 1], o[db][4 * v4 + 2], o[db][4 * v4 + 3]);
    }
}

bool diff_attention_heads_takes(const DiffAttnArgs& a) {
  return diff_attention_tiles_takes(a) && a.max_qlen == 1 && a.Hq / a.Hkv <= 32;
}

// Chunks of the context (multiples of 64 keys) so that the launch has about four blocks a CU.
void diff_attention_heads_plan(const DiffAttnArgs& a, int* chunk, int* n_chunks) {
  const int blocks = a.T * a.Hkv;
  const int want = (4 * device_cu_count() + blocks - 1) / blocks;
  int per = (a.max_kv_len + want - 1) / want;
  // (at least 256 keys a chunk: every chunk leaves two records a head for the merge to read)
  per = ((per < 256 ? 256 : per) + 63) / 64 * 64;
  *chunk = per;
  *n_chunks = (a.max_kv_len + per - 1) / per;
}

template <int KS, int DB>
static int launch_heads(const DiffAttnArgs& a, int chunk, int n_chunks, hipStream_t stream) {
  constexpr int DP = 16 * KS, VP = 32 * DB;
  const size_t lds = (64 * (2 * DP + 8) + 64 * (VP + 8)) * sizeof(unsigned short);
  auto kern = diff_attention_heads_kernel<KS, DB>;
  if (lds > 64 * 1024) {
    static bool raised = false;
    if (!raised) {
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return set_error(-2, "diff_attention: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
      raised = true;
    }
  }
  kern<<<dim3(a.T, a.Hkv, n_chunks), 256, lds, stream>>>(a, chunk, n_chunks);
  NINFER_LAUNCH_CHECK();
  return diff_attention_merge(a, 2 * n_chunks, stream);
}

int diff_attention_heads(const DiffAttnArgs& a, int chunk, int n_chunks, hipStream_t stream) {
  NINFER_REQUIRE(a.workspace && a.workspace_floats >= (int64_t)a.T * a.Hq * 2 * n_chunks * (4 + 2 * a.vdim),
                 "diff_attention: the workspace is too small for %d chunks", n_chunks);
  const int db = (a.vdim + 31) / 32;
  const int ks = a.dim <= 32 ? 2 : a.dim <= 48 ? 3 : a.dim <= 64 ? 4 : a.dim <= 96 ? 6 : 8;
#define NINFER_DIFF_HEADS(KS_)                                                  \
  switch (db) {                                                                 \
    case 1: return launch_heads<KS_, 1>(a, chunk, n_chunks, stream);            \
    case 2: return launch_heads<KS_, 2>(a, chunk, n_chunks, stream);            \
    case 3: return launch_heads<KS_, 3>(a, chunk, n_chunks, stream);            \
    default: return launch_heads<KS_, 4>(a, chunk, n_chunks, stream);           \
  }
  switch (ks) {
    case 2: NINFER_DIFF_HEADS(2)
    case 3: NINFER_DIFF_HEADS(3)
    case 4: NINFER_DIFF_HEADS(4)
    case 6: NINFER_DIFF_HEADS(6)
    default: NINFER_DIFF_HEADS(8)
  }
#undef NINFER_DIFF_HEADS
}

template <int KS, int DB>
static int launch_tiles(const DiffAttnArgs& a, int first_seq, hipStream_t stream) {
  const int hpg = a.Hq / a.Hkv;
  const int HB = hpg % 2 == 0 ? 2 : 1;
  const int RT = 32 * (2 / HB);
  constexpr int DP = 16 * KS, VP = 32 * DB;
  const size_t lds = 2 * (64 * (2 * DP + 8) + 64 * (VP + 8)) * sizeof(unsigned short);
  auto kern = diff_attention_tiles_kernel<KS, DB>;
  if (lds > 64 * 1024) {
    static bool raised = false;   // per instantiation
    if (!raised) {
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return set_error(-2, "diff_attention: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
      raised = true;
    }
  }
  // (requests before first_seq bring one row each)
  dim3 grid((a.T - first_seq) / RT + a.S - first_seq, a.Hkv * (hpg / HB));
  kern<<<grid, 256, lds, stream>>>(a, HB, first_seq);
  NINFER_LAUNCH_CHECK();
  return 0;
}

int diff_attention_tiles(const DiffAttnArgs& a, int first_seq, hipStream_t stream) {
  const int db = (a.vdim + 31) / 32;
  const int ks = a.dim <= 32 ? 2 : a.dim <= 48 ? 3 : a.dim <= 64 ? 4 : a.dim <= 96 ? 6 : 8;
#define NINFER_DIFF_TILES(KS_)                                   \
  switch (db) {                                                  \
    case 1: return launch_tiles<KS_, 1>(a, first_seq, stream);              \
    case 2: return launch_tiles<KS_, 2>(a, first_seq, stream);              \
    case 3: return launch_tiles<KS_, 3>(a, first_seq, stream);              \
    default: return launch_tiles<KS_, 4>(a, first_seq, stream);             \
  }
  switch (ks) {
    case 2: NINFER_DIFF_TILES(2)
    case 3: NINFER_DIFF_TILES(3)
    case 4: NINFER_DIFF_TILES(4)
    case 6: NINFER_DIFF_TILES(6)
    default: NINFER_DIFF_TILES(8)
  }
#undef NINFER_DIFF_TILES
}

}  // namespace ninfer
