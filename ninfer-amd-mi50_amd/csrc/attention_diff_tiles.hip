// Differential attention for prompt portions on the matrix cores (bf16 rows and cache).
//
// A block of four waves owns one kv head and a tile of rows of one request: every wave 32
// rows of one query head (HB query heads of the kv head side by side, 4 / HB groups of 32
// rows), so that all waves meet the same keys and values. These are walked in tiles of 64
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
// with the contraction index numbered as the lanes hold it. Both maps read the same value
// fragments. At the end o = O1 / l1 - lambda O2 / l2, the head's norm over its value columns,
// the factor, the store.
// Keys that do not exist (beyond the tile's last row) load the last row's key in their place:
// they are masked, and their values must be finite since 0 x NaN is not 0.
#include "attention_diff.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) short4v lds_short4;

constexpr float kLog2e = 1.44269504088896f;

template <int KS, int DB>
__global__ __launch_bounds__(256) void diff_attention_tiles_kernel(DiffAttnArgs a, int HB) {
  constexpr int DP = 16 * KS, KROW = 2 * DP + 8, VP = 32 * DB, VROW = VP + 8;
  constexpr int TILE = 64 * KROW + 64 * VROW;   // elements of one buffer
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
    int idx = blockIdx.x;
    for (int s = 0; s < a.S; ++s) {
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
  for (int i = tid; i < 2 * TILE / 8; i += 256) ((uint4*)lds)[i] = make_uint4(0, 0, 0, 0);

  // this thread's pieces of a tile (16 bytes each): key row, column in global memory and in LDS
  int k_key[KS], k_src[KS], k_dst[KS], v_key[DB], v_src[DB];
  {
    const int cpk = kd / 8, cpv = vdim / 8;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int p = i * 256 + tid;
      k_key[i] = p < 64 * cpk ? p / cpk : -1;
      k_src[i] = (p % cpk) * 8;
      k_dst[i] = k_src[i] < dim ? k_src[i] : DP + k_src[i] - dim;
    }
#pragma unroll
    for (int i = 0; i < DB; ++i) {
      const int p = i * 256 + tid;
      v_key[i] = p < 64 * cpv ? p / cpv : -1;
      v_src[i] = (p % cpv) * 8;
    }
  }
  uint4 kreg[KS], vreg[DB];
  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      if (k_key[i] < 0) continue;
      const int j = min(k0 + k_key[i], pos_last);
      const int64_t at = ((int64_t)bt[j >> ps_shift] * a.Hkv + g) * a.page_size + (j & ps_mask);
      kreg[i] = *(const uint4*)(kpool + at * kd + k_src[i]);
    }
#pragma unroll
    for (int i = 0; i < DB; ++i) {
      if (v_key[i] < 0) continue;
      const int j = min(k0 + v_key[i], pos_last);
      const int64_t at = ((int64_t)bt[j >> ps_shift] * a.Hkv + g) * a.page_size + (j & ps_mask);
      vreg[i] = *(const uint4*)(vpool + at * vdim + v_src[i]);
    }
  };
  auto store_tile = [&](int buf) {
    unsigned short* ks = lds + buf * TILE;
    unsigned short* vs = ks + 64 * KROW;
#pragma unroll
    for (int i = 0; i < KS; ++i)
      if (k_key[i] >= 0) *(uint4*)(ks + k_key[i] * KROW + k_dst[i]) = kreg[i];
#pragma unroll
    for (int i = 0; i < DB; ++i)
      if (v_key[i] >= 0) *(uint4*)(vs + v_key[i] * VROW + v_src[i]) = vreg[i];
  };

  // this lane's queries (B operand): row c of the wave, dims 16 ks + 8 hi .. + 7 of each map
  const bool wave_live = rs * 32 < n_rows;
  const int q_local = rs * 32 + c;
  const bool q_valid = q_local < n_rows;
  const int q_pos = pos_first + q_local;
  const int wave_last = pos_first + min(rs * 32 + 31, n_rows - 1);
  bf16x8 qf[2][KS];
  {
    const unsigned short* qr = (const unsigned short*)a.qkv +
                               (int64_t)(row0 + (q_valid ? q_local : 0)) * a.q_stride + h * kd;
#pragma unroll
    for (int mp = 0; mp < 2; ++mp)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d = 16 * ks + 8 * hi;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (d < dim) v = *(const uint4*)(qr + mp * dim + d);
        qf[mp][ks] = __builtin_bit_cast(bf16x8, v);
      }
  }
  // scores in units of log 2: (q . k) qscale, capped, times log2(e)
  const float qscale = a.scale * (a.t_coef == 0.f ? 1.f
                                  : 1.f + a.t_coef * logf((float)((q_pos + 1) / a.t_every) + 1.f));
  const bool capped = a.cap > 0.f;
  const float pre = capped ? qscale / a.cap * 2.f * kLog2e : qscale * kLog2e;
  const float cap2 = a.cap * kLog2e;

  f32x16 o[2][DB];
#pragma unroll
  for (int mp = 0; mp < 2; ++mp)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[mp][db][v] = 0.f;
  float m[2] = {-1e30f, -1e30f}, l[2] = {0.f, 0.f};

  // the transposing read's address of this lane inside a value tile: lane s of a group of 16
  // fetches key s / 4 (+ 4 hi), value columns 16 (group % 2) + 4 (s % 4) .. + 3
  const int s16 = lane & 15, q4 = lane >> 4;
  const int v_lane = (4 * hi + s16 / 4) * VROW + 16 * (q4 & 1) + 4 * (s16 & 3);

  load_tile(0);
  __syncthreads();   // the zeros are written
  const int n_kt = pos_last / 64 + 1;
  for (int kt = 0; kt < n_kt; ++kt) {
    const int k0 = kt * 64, buf = kt & 1;
    store_tile(buf);
    __syncthreads();
    if (kt + 1 < n_kt) load_tile(k0 + 64);
    if (!wave_live || k0 > wave_last) continue;
    const unsigned short* ks_ = lds + buf * TILE;
    const unsigned short* vs_ = ks_ + 64 * KROW;
    const bool masked = k0 + 63 > pos_first + rs * 32;   // some row of the wave does not see every key
    bf16x8 pf[2][2][2];
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
      f32x16 s[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) s[kb][v] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 kf = *(const bf16x8*)(ks_ + (32 * kb + c) * KROW + mp * DP + 16 * ks + 8 * hi);
          s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[mp][ks], s[kb], 0, 0, 0);
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
      const float m_new = fmaxf(m[mp], mx);
      if (__any(m_new > m[mp])) {
        const float alpha = __builtin_amdgcn_exp2f(m[mp] - m_new);
        l[mp] *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[mp][db][v] *= alpha;
        m[mp] = m_new;
      }
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh)
#pragma unroll
          for (int jj = 0; jj < 8; ++jj) {
            const float p = __builtin_amdgcn_exp2f(s[kb][8 * hh + jj] - m[mp]);
            psum += p;
            pf[mp][kb][hh][jj] = (__bf16)p;
          }
      l[mp] += psum + __shfl_xor(psum, 32, 64);
    }
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x8 vf[2][2];
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
          vf[kb][hh] = __builtin_bit_cast(bf16x8, both);
        }
#pragma unroll
      for (int mp = 0; mp < 2; ++mp)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int hh = 0; hh < 2; ++hh)
            o[mp][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[kb][hh], pf[mp][kb][hh], o[mp][db], 0, 0, 0);
    }
  }
  if (!wave_live) return;
  // o = O1 / l1 - lambda O2 / l2; the norm over the head's value columns; the store. Lane
  // holds, for row c, value columns 32 db + 8 (v / 4) + 4 hi + v % 4.
  const float i1 = 1.f / l[0], i2 = a.lambda / l[1];
  float ss = 0.f;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float x = o[0][db][v] * i1 - o[1][db][v] * i2;
      o[0][db][v] = x;
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
        for (int e = 0; e < 4; ++e) w.b[e] = (__bf16)(o[0][db][4 * v4 + e] * r);
        *(uint2*)(orow + col) = w.u;
      }
    }
}

bool diff_attention_tiles_takes(const DiffAttnArgs& a) {
  return a.dtype == kBF16 && a.dim % 8 == 0 && a.vdim % 8 == 0 && a.dim <= 128 && a.vdim <= 128 &&
         a.q_stride % 8 == 0 && (a.page_size & (a.page_size - 1)) == 0;
}

template <int KS, int DB>
static int launch_tiles(const DiffAttnArgs& a, hipStream_t stream) {
  const int hpg = a.Hq / a.Hkv;
  const int HB = hpg % 4 == 0 ? 4 : (hpg % 2 == 0 ? 2 : 1);
  const int RT = 32 * (4 / HB);
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
  dim3 grid(a.T / RT + a.S, a.Hkv * (hpg / HB));
  kern<<<grid, 256, lds, stream>>>(a, HB);
  NINFER_LAUNCH_CHECK();
  return 0;
}

int diff_attention_tiles(const DiffAttnArgs& a, hipStream_t stream) {
  const int db = (a.vdim + 31) / 32;
  const int ks = a.dim <= 32 ? 2 : a.dim <= 48 ? 3 : a.dim <= 64 ? 4 : a.dim <= 96 ? 6 : 8;
#define NINFER_DIFF_TILES(KS_)                                   \
  switch (db) {                                                  \
    case 1: return launch_tiles<KS_, 1>(a, stream);              \
    case 2: return launch_tiles<KS_, 2>(a, stream);              \
    case 3: return launch_tiles<KS_, 3>(a, stream);              \
    default: return launch_tiles<KS_, 4>(a, stream);             \
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
