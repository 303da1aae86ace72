// Differential attention over the paged cache (see attention_diff.h for what it computes):
// the write of keys and values into pages, the plain kernel (one wave per row and query
// head, both maps at once; the 32-bit path, sizes the matrix-core kernel refuses, and single
// rows with their contexts cut into chunks), and the merge of such chunks.
//
// Keys are walked in tiles of 64 aligned to absolute positions with an online softmax per
// map, so without chunks the order of every sum depends on the row's own position only.
// Scores, both softmaxes, the difference and the head's norm are 32-bit.
#include "attention_diff.h"

namespace ninfer {

constexpr int kMaxVPerLane = 8;   // value sizes up to 512

// temp(p) = 1 + coef ln(floor((p + 1) / every) + 1)
__device__ __forceinline__ float query_temperature(int pos, float coef, int every) {
  if (coef == 0.f) return 1.f;
  return 1.f + coef * logf((float)((pos + 1) / every) + 1.f);
}

// k and v of every row into the request's pages.
template <typename T>
__global__ void diff_kv_write_kernel(DiffAttnArgs a) {
  const int t = blockIdx.x;
  const int pos = a.positions[t];
  const int page = a.block_table[(int64_t)a.row_seq[t] * a.bt_stride + pos / a.page_size];
  const int slot = pos % a.page_size;
  const int kd = 2 * a.dim;
  const T* row = (const T*)a.qkv + (int64_t)t * a.q_stride + a.Hq * kd;
  T* kp = (T*)a.kpool;
  T* vp = (T*)a.vpool;
  const int nk = a.Hkv * kd, nv = a.Hkv * a.vdim;
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int g = i / kd, d = i % kd;
    kp[(((int64_t)page * a.Hkv + g) * a.page_size + slot) * kd + d] = row[i];
  }
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const int g = i / a.vdim, d = i % a.vdim;
    vp[(((int64_t)page * a.Hkv + g) * a.page_size + slot) * a.vdim + d] = row[nk + i];
  }
}

// o = a1 / l1 - lambda a2 / l2 over the lane's value columns, the head's norm, the store.
template <typename T>
__device__ __forceinline__ void diff_finish(const DiffAttnArgs& a, const float* acc1,
                                            const float* acc2, float l1, float l2, T* orow,
                                            int lane) {
  const float i1 = 1.f / l1, i2 = a.lambda / l2;
  float o[kMaxVPerLane];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxVPerLane; ++i) {
    const int d = lane + i * 64;
    o[i] = d < a.vdim ? acc1[i] * i1 - acc2[i] * i2 : 0.f;
    ss += o[i] * o[i];
  }
  float r = a.out_scale;
  if (a.eps >= 0.f) r *= 1.f / sqrtf(wave_sum(ss) / (float)a.vdim + a.eps);
#pragma unroll
  for (int i = 0; i < kMaxVPerLane; ++i) {
    const int d = lane + i * 64;
    if (d < a.vdim) orow[d] = from_f32<T>(o[i] * r);
  }
}

// One wave per (row, query head, chunk of the context). n_chunks == 1: the whole context,
// result written to out; else keys [c chunk, (c + 1) chunk) and partial results
// {m1, l1, m2, l2, acc1[vdim], acc2[vdim]} into the workspace.
template <typename T>
__global__ __launch_bounds__(64) void diff_attention_plain_kernel(DiffAttnArgs a, int chunk,
                                                                  int n_chunks) {
  extern __shared__ float smem[];
  const int kd = 2 * a.dim;
  float* q_s = smem;                  // [2 dim]
  float* p1_s = q_s + kd;             // [64]
  float* p2_s = p1_s + 64;            // [64]
  int64_t* off_s = (int64_t*)(p2_s + 64 + ((kd & 1) ? 1 : 0));   // [64] element offset of each value row

  const int t = blockIdx.x, h = blockIdx.y, c = blockIdx.z, lane = threadIdx.x;
  const int g = h / (a.Hq / a.Hkv);
  const int pos = a.positions[t];
  const int* bt = a.block_table + (int64_t)a.row_seq[t] * a.bt_stride;
  const int first = n_chunks > 1 ? c * chunk : 0;
  const int last = n_chunks > 1 ? min(pos, first + chunk - 1) : pos;
  const float qscale = a.scale * query_temperature(pos, a.t_coef, a.t_every);
  const T* kpool = (const T*)a.kpool;
  const T* vpool = (const T*)a.vpool;

  const T* qr = (const T*)a.qkv + (int64_t)t * a.q_stride + h * kd;
  for (int d = lane; d < kd; d += 64) q_s[d] = to_f32(qr[d]);
  __syncthreads();

  float m1 = -INFINITY, l1 = 0.f, m2 = -INFINITY, l2 = 0.f;
  float acc1[kMaxVPerLane], acc2[kMaxVPerLane];
#pragma unroll
  for (int i = 0; i < kMaxVPerLane; ++i) acc1[i] = acc2[i] = 0.f;

  for (int tile = first; tile <= last; tile += 64) {   // chunks are multiples of 64
    const int j = tile + lane;
    const bool valid = j <= last;
    float s1 = -INFINITY, s2 = -INFINITY;
    int64_t voff = 0;
    if (valid) {
      const int page = bt[j / a.page_size];
      const int64_t at = ((int64_t)page * a.Hkv + g) * a.page_size + (j % a.page_size);
      voff = at * a.vdim;
      const T* kr = kpool + at * kd;
      float d1 = 0.f, d2 = 0.f;
      for (int d = 0; d < a.dim; ++d) d1 = fmaf(q_s[d], to_f32(kr[d]), d1);
      for (int d = 0; d < a.dim; ++d) d2 = fmaf(q_s[a.dim + d], to_f32(kr[a.dim + d]), d2);
      s1 = d1 * qscale;
      s2 = d2 * qscale;
      if (a.cap > 0.f) {
        s1 = a.cap * tanhf(s1 / a.cap);
        s2 = a.cap * tanhf(s2 / a.cap);
      }
    }
    const float n1 = fmaxf(m1, wave_max(s1)), n2 = fmaxf(m2, wave_max(s2));
    const float p1 = valid ? expf(s1 - n1) : 0.f, p2 = valid ? expf(s2 - n2) : 0.f;
    const float al1 = expf(m1 - n1), al2 = expf(m2 - n2);   // 0 on the first tile
    l1 = l1 * al1 + wave_sum(p1);
    l2 = l2 * al2 + wave_sum(p2);
    m1 = n1;
    m2 = n2;
    p1_s[lane] = p1;
    p2_s[lane] = p2;
    off_s[lane] = voff;
    __syncthreads();
    const int n_keys = min(64, last - tile + 1);
#pragma unroll
    for (int i = 0; i < kMaxVPerLane; ++i) {
      const int d = lane + i * 64;
      if (d < a.vdim) {
        float x1 = acc1[i] * al1, x2 = acc2[i] * al2;
        for (int jj = 0; jj < n_keys; ++jj) {
          const float v = to_f32(vpool[off_s[jj] + d]);
          x1 = fmaf(p1_s[jj], v, x1);
          x2 = fmaf(p2_s[jj], v, x2);
        }
        acc1[i] = x1;
        acc2[i] = x2;
      }
    }
    __syncthreads();
  }
  if (n_chunks == 1) {
    diff_finish<T>(a, acc1, acc2, l1, l2, (T*)a.out + ((int64_t)t * a.Hq + h) * a.vdim, lane);
    return;
  }
  float* part = a.workspace + (((int64_t)t * a.Hq + h) * n_chunks + c) * (4 + 2 * a.vdim);
  if (lane == 0) {
    part[0] = m1;
    part[1] = l1;
    part[2] = m2;
    part[3] = l2;
  }
#pragma unroll
  for (int i = 0; i < kMaxVPerLane; ++i) {
    const int d = lane + i * 64;
    if (d < a.vdim) {
      part[4 + d] = acc1[i];
      part[4 + a.vdim + d] = acc2[i];
    }
  }
}

// The records of a row and head put together by a block of four waves (a record whose l is 0
// counts for nothing: a chunk that starts beyond the row's position, a wave that met no key).
// The threads first take a record each: the largest m of each map, then every record's weight
// exp(m - M) into LDS and the sum of the weighted l; then wave w adds up the weighted records
// w, w + 4, ... over its lanes' value columns, and the first wave adds the four sums and
// finishes the head.
template <typename T>
__global__ __launch_bounds__(256) void diff_attention_merge_kernel(DiffAttnArgs a, int n_records) {
  extern __shared__ float w_s[];          // [2][n_records], then 16 for reductions, then [4][2][vdim]
  float* red = w_s + 2 * n_records;
  float* acc_s = red + 16;
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int stride = 4 + 2 * a.vdim;
  const float* part = a.workspace + ((int64_t)t * a.Hq + h) * n_records * stride;
  float m1 = -INFINITY, m2 = -INFINITY;
  for (int c = tid; c < n_records; c += 256) {
    const float* r = part + (int64_t)c * stride;
    if (r[1] > 0.f) m1 = fmaxf(m1, r[0]);
    if (r[3] > 0.f) m2 = fmaxf(m2, r[2]);
  }
  m1 = wave_max(m1);
  m2 = wave_max(m2);
  if (lane == 0) {
    red[w] = m1;
    red[4 + w] = m2;
  }
  __syncthreads();
  m1 = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  m2 = fmaxf(fmaxf(red[4], red[5]), fmaxf(red[6], red[7]));
  float l1 = 0.f, l2 = 0.f;
  for (int c = tid; c < n_records; c += 256) {
    const float* r = part + (int64_t)c * stride;
    const float w1 = r[1] > 0.f ? expf(r[0] - m1) : 0.f, w2 = r[3] > 0.f ? expf(r[2] - m2) : 0.f;
    w_s[c] = w1;
    w_s[n_records + c] = w2;
    l1 += w1 > 0.f ? w1 * r[1] : 0.f;
    l2 += w2 > 0.f ? w2 * r[3] : 0.f;
  }
  l1 = wave_sum(l1);
  l2 = wave_sum(l2);
  if (lane == 0) {
    red[8 + w] = l1;
    red[12 + w] = l2;
  }
  __syncthreads();
  l1 = (red[8] + red[9]) + (red[10] + red[11]);
  l2 = (red[12] + red[13]) + (red[14] + red[15]);
  float acc1[kMaxVPerLane], acc2[kMaxVPerLane];
#pragma unroll
  for (int i = 0; i < kMaxVPerLane; ++i) acc1[i] = acc2[i] = 0.f;
#pragma unroll 4
  for (int c = w; c < n_records; c += 4) {
    const float* p = part + (int64_t)c * stride + 4;
    const float w1 = w_s[c], w2 = w_s[n_records + c];
#pragma unroll
    for (int i = 0; i < kMaxVPerLane; ++i) {
      const int d = lane + i * 64;
      if (d < a.vdim) {
        // (a record that counts for nothing may hold anything: it does not enter the sum)
        const float x1 = p[d], x2 = p[a.vdim + d];
        acc1[i] += w1 > 0.f ? w1 * x1 : 0.f;
        acc2[i] += w2 > 0.f ? w2 * x2 : 0.f;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxVPerLane; ++i) {
    const int d = lane + i * 64;
    if (d < a.vdim) {
      acc_s[(w * 2) * a.vdim + d] = acc1[i];
      acc_s[(w * 2 + 1) * a.vdim + d] = acc2[i];
    }
  }
  __syncthreads();
  if (w != 0) return;
#pragma unroll
  for (int i = 0; i < kMaxVPerLane; ++i) {
    const int d = lane + i * 64;
    if (d < a.vdim) {
      acc1[i] = (acc_s[d] + acc_s[2 * a.vdim + d]) + (acc_s[4 * a.vdim + d] + acc_s[6 * a.vdim + d]);
      acc2[i] = (acc_s[a.vdim + d] + acc_s[3 * a.vdim + d]) + (acc_s[5 * a.vdim + d] + acc_s[7 * a.vdim + d]);
    }
  }
  diff_finish<T>(a, acc1, acc2, l1, l2, (T*)a.out + ((int64_t)t * a.Hq + h) * a.vdim, lane);
}

// Single rows (decode steps) in bfloat16: a block of four waves owns one row, HB query heads of
// one kv head and one chunk of the context, so that keys and values are read once for all of
// these heads. The waves take the chunk's tiles of 64 keys in turn. Per tile a lane owns a
// key: its row is loaded in 16-byte pieces and multiplied with the queries of all HB heads and
// both maps (32-bit, from LDS); the online softmax of each head and map runs across the wave;
// then a lane owns value columns lane + 64 v and adds up p x value over the tile's keys for
// every head and map. The waves' sums are put together through LDS, and the block writes the
// result (one chunk) or its partial sums (the merge kernel's format).
template <int HB, int VPL>
__global__ __launch_bounds__(256) void diff_attention_rows_kernel(DiffAttnArgs a, int chunk,
                                                                  int n_chunks) {
  constexpr int HM = 2 * HB;   // (head, map) pairs
  extern __shared__ float smem[];
  const int kd = 2 * a.dim, dim = a.dim, vdim = a.vdim;
  float* q_s = smem;                                   // [HB][2 dim]
  float* p_s = q_s + HB * kd;                          // [4][HM][64]
  float* ml_s = p_s + 4 * HM * 64;                     // [4][HM][2]
  float* acc_s = ml_s + 4 * HM * 2;                    // [4][HM][VPL * 64]
  int64_t* off_s = (int64_t*)(acc_s + 4 * HM * VPL * 64);   // [4][64]

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int t = blockIdx.x, c = blockIdx.z;
  const int hpg = a.Hq / a.Hkv;
  const int g = blockIdx.y / (hpg / HB);
  const int h0 = g * hpg + (blockIdx.y % (hpg / HB)) * HB;
  const int pos = a.positions[t];
  const int* bt = a.block_table + (int64_t)a.row_seq[t] * a.bt_stride;
  const int first = n_chunks > 1 ? c * chunk : 0;
  const int last = n_chunks > 1 ? min(pos, first + chunk - 1) : pos;
  const float qscale = a.scale * query_temperature(pos, a.t_coef, a.t_every);
  const bf16* kpool = (const bf16*)a.kpool;
  const bf16* vpool = (const bf16*)a.vpool;

  const bf16* qr = (const bf16*)a.qkv + (int64_t)t * a.q_stride + h0 * kd;
  for (int i = tid; i < HB * kd; i += 256) q_s[i] = to_f32(qr[i]);
  __syncthreads();

  float m[HM], l[HM], acc[HM][VPL];
#pragma unroll
  for (int i = 0; i < HM; ++i) {
    m[i] = -1e30f;
    l[i] = 0.f;
#pragma unroll
    for (int v = 0; v < VPL; ++v) acc[i][v] = 0.f;
  }
  float* my_p = p_s + w * HM * 64;
  int64_t* my_off = off_s + w * 64;

  for (int tile = first + 64 * w; tile <= last; tile += 256) {
    const int j = tile + lane;
    const bool valid = j <= last;
    const int jc = min(j, last);   // a key that is not there: the last one's row in its place
    const int64_t at = ((int64_t)bt[jc / a.page_size] * a.Hkv + g) * a.page_size + jc % a.page_size;
    typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
    const uint4v* kr = (const uint4v*)(kpool + at * kd);
    float dots[HM];
#pragma unroll
    for (int i = 0; i < HM; ++i) dots[i] = 0.f;
#pragma unroll
    for (int mp = 0; mp < 2; ++mp)
      for (int d8 = 0; d8 < dim / 8; ++d8) {
        const uint4v kk = stream_load(kr + mp * (dim / 8) + d8);
        float kf[8];
        kf[0] = __uint_as_float(kk.x << 16); kf[1] = __uint_as_float(kk.x & 0xffff0000u);
        kf[2] = __uint_as_float(kk.y << 16); kf[3] = __uint_as_float(kk.y & 0xffff0000u);
        kf[4] = __uint_as_float(kk.z << 16); kf[5] = __uint_as_float(kk.z & 0xffff0000u);
        kf[6] = __uint_as_float(kk.w << 16); kf[7] = __uint_as_float(kk.w & 0xffff0000u);
#pragma unroll
        for (int hb = 0; hb < HB; ++hb) {
          const float4 qa = *(const float4*)(q_s + hb * kd + mp * dim + d8 * 8);
          const float4 qb = *(const float4*)(q_s + hb * kd + mp * dim + d8 * 8 + 4);
          float s = dots[2 * hb + mp];
          s = fmaf(qa.x, kf[0], s); s = fmaf(qa.y, kf[1], s); s = fmaf(qa.z, kf[2], s); s = fmaf(qa.w, kf[3], s);
          s = fmaf(qb.x, kf[4], s); s = fmaf(qb.y, kf[5], s); s = fmaf(qb.z, kf[6], s); s = fmaf(qb.w, kf[7], s);
          dots[2 * hb + mp] = s;
        }
      }
    float alpha[HM];
#pragma unroll
    for (int i = 0; i < HM; ++i) {
      float s = dots[i] * qscale;
      if (a.cap > 0.f) s = a.cap * tanhf(s / a.cap);
      if (!valid) s = -INFINITY;
      const float m_new = fmaxf(m[i], wave_max(s));
      const float p = valid ? expf(s - m_new) : 0.f;
      alpha[i] = expf(m[i] - m_new);
      l[i] = l[i] * alpha[i] + wave_sum(p);
      m[i] = m_new;
      my_p[i * 64 + lane] = p;
    }
    my_off[lane] = at * vdim;
    __builtin_amdgcn_wave_barrier();   // the wave's own writes above are read below, in order
    const int n_keys = min(64, last - tile + 1);
#pragma unroll
    for (int i = 0; i < HM; ++i)
#pragma unroll
      for (int v = 0; v < VPL; ++v) acc[i][v] *= alpha[i];
    for (int jj = 0; jj < n_keys; ++jj) {
      const bf16* vr = vpool + my_off[jj];
      float val[VPL];
#pragma unroll
      for (int v = 0; v < VPL; ++v) val[v] = lane + 64 * v < vdim ? to_f32(vr[lane + 64 * v]) : 0.f;
#pragma unroll
      for (int i = 0; i < HM; ++i) {
        const float p = my_p[i * 64 + jj];
#pragma unroll
        for (int v = 0; v < VPL; ++v) acc[i][v] = fmaf(p, val[v], acc[i][v]);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // the four waves' sums put together: wave hb finishes head hb
  if (lane == 0)
    for (int i = 0; i < HM; ++i) {
      ml_s[(w * HM + i) * 2] = m[i];
      ml_s[(w * HM + i) * 2 + 1] = l[i];
    }
#pragma unroll
  for (int i = 0; i < HM; ++i)
#pragma unroll
    for (int v = 0; v < VPL; ++v) acc_s[((w * HM + i) * VPL + v) * 64 + lane] = acc[i][v];
  __syncthreads();
  if (w >= HB) return;
  float fm[2], fl[2], facc[2][kMaxVPerLane];
#pragma unroll
  for (int mp = 0; mp < 2; ++mp) {
    const int i = 2 * w + mp;
    float mm = -1e30f;
    for (int x = 0; x < 4; ++x) mm = fmaxf(mm, ml_s[(x * HM + i) * 2]);
    float ll = 0.f;
#pragma unroll
    for (int v = 0; v < kMaxVPerLane; ++v) facc[mp][v] = 0.f;
    for (int x = 0; x < 4; ++x) {
      const float f = expf(ml_s[(x * HM + i) * 2] - mm);
      ll += f * ml_s[(x * HM + i) * 2 + 1];
#pragma unroll
      for (int v = 0; v < VPL; ++v) facc[mp][v] = fmaf(f, acc_s[((x * HM + i) * VPL + v) * 64 + lane], facc[mp][v]);
    }
    fm[mp] = mm;
    fl[mp] = ll;
  }
  const int h = h0 + w;
  if (n_chunks == 1) {
    diff_finish<bf16>(a, facc[0], facc[1], fl[0], fl[1], (bf16*)a.out + ((int64_t)t * a.Hq + h) * vdim, lane);
    return;
  }
  float* part = a.workspace + (((int64_t)t * a.Hq + h) * n_chunks + c) * (4 + 2 * vdim);
  if (lane == 0) {
    part[0] = fm[0];
    part[1] = fl[0];
    part[2] = fm[1];
    part[3] = fl[1];
  }
#pragma unroll
  for (int v = 0; v < VPL; ++v) {
    const int d = lane + 64 * v;
    if (d < vdim) {
      part[4 + d] = facc[0][v];
      part[4 + vdim + d] = facc[1][v];
    }
  }
}

static bool diff_rows_takes(const DiffAttnArgs& a) {
  return a.dtype == kBF16 && a.max_qlen == 1 && !a.force_plain && a.dim % 8 == 0 && a.vdim <= 256 &&
         a.q_stride % 8 == 0;
}

static int diff_rows_heads(const DiffAttnArgs& a) {
  const int hpg = a.Hq / a.Hkv;
  return hpg % 4 == 0 ? 4 : (hpg % 2 == 0 ? 2 : 1);
}

template <int HB>
static int launch_rows(const DiffAttnArgs& a, int chunk, int n_chunks, hipStream_t stream) {
  const int vpl = (a.vdim + 63) / 64;
  const size_t lds = (size_t)(HB * 2 * a.dim + 4 * 2 * HB * 64 + 4 * 2 * HB * 2 + 4 * 2 * HB * vpl * 64) * sizeof(float) +
                     4 * 64 * sizeof(int64_t);
  dim3 grid(a.T, a.Hkv * (a.Hq / a.Hkv / HB), n_chunks);
  switch (vpl) {
    case 1: diff_attention_rows_kernel<HB, 1><<<grid, 256, lds, stream>>>(a, chunk, n_chunks); break;
    case 2: diff_attention_rows_kernel<HB, 2><<<grid, 256, lds, stream>>>(a, chunk, n_chunks); break;
    case 3: diff_attention_rows_kernel<HB, 3><<<grid, 256, lds, stream>>>(a, chunk, n_chunks); break;
    default: diff_attention_rows_kernel<HB, 4><<<grid, 256, lds, stream>>>(a, chunk, n_chunks); break;
  }
  NINFER_LAUNCH_CHECK();
  if (n_chunks > 1) {
    diff_attention_merge_kernel<bf16><<<dim3(a.T, a.Hq), 256, (2 * n_chunks + 16 + 8 * a.vdim) * sizeof(float), stream>>>(a, n_chunks);
    NINFER_LAUNCH_CHECK();
  }
  return 0;
}

static int diff_attention_rows(const DiffAttnArgs& a, int chunk, int n_chunks, hipStream_t stream) {
  switch (diff_rows_heads(a)) {
    case 4: return launch_rows<4>(a, chunk, n_chunks, stream);
    case 2: return launch_rows<2>(a, chunk, n_chunks, stream);
    default: return launch_rows<1>(a, chunk, n_chunks, stream);
  }
}

int diff_attention_plain(const DiffAttnArgs& a, int chunk, int n_chunks, hipStream_t stream) {
  const size_t lds = (2 * a.dim + 128 + 2) * sizeof(float) + 64 * sizeof(int64_t);
  dim3 grid(a.T, a.Hq, n_chunks);
  if (a.dtype == kF32) {
    diff_attention_plain_kernel<float><<<grid, 64, lds, stream>>>(a, chunk, n_chunks);
    if (n_chunks > 1) diff_attention_merge_kernel<float><<<dim3(a.T, a.Hq), 256, (2 * n_chunks + 16 + 8 * a.vdim) * sizeof(float), stream>>>(a, n_chunks);
  } else {
    diff_attention_plain_kernel<bf16><<<grid, 64, lds, stream>>>(a, chunk, n_chunks);
    if (n_chunks > 1) diff_attention_merge_kernel<bf16><<<dim3(a.T, a.Hq), 256, (2 * n_chunks + 16 + 8 * a.vdim) * sizeof(float), stream>>>(a, n_chunks);
  }
  NINFER_LAUNCH_CHECK();
  return 0;
}

int diff_attention_merge(const DiffAttnArgs& a, int n_records, hipStream_t stream) {
  if (a.dtype == kF32) diff_attention_merge_kernel<float><<<dim3(a.T, a.Hq), 256, (2 * n_records + 16 + 8 * a.vdim) * sizeof(float), stream>>>(a, n_records);
  else diff_attention_merge_kernel<bf16><<<dim3(a.T, a.Hq), 256, (2 * n_records + 16 + 8 * a.vdim) * sizeof(float), stream>>>(a, n_records);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// Single rows (a decode step): how the contexts are cut so that the launch fills the GPU.
static void diff_chunks(const DiffAttnArgs& a, int* chunk, int* n_chunks) {
  *chunk = 0;
  *n_chunks = 1;
  if (a.dtype != kBF16 || a.max_qlen != 1 || a.force_plain) return;
  int per;
  if (diff_rows_takes(a)) {
    // blocks of four waves, each wave a tile of 64 keys at a time: two blocks a CU
    const int blocks = a.T * (a.Hq / diff_rows_heads(a));
    const int want = (2 * device_cu_count() + blocks - 1) / blocks;
    per = (a.max_kv_len + want - 1) / want;
  } else {
    const int waves = a.T * a.Hq;
    const int want = (8 * device_cu_count() + waves - 1) / waves;   // eight waves a CU
    per = (a.max_kv_len + want - 1) / want;
  }
  per = ((per < 256 ? 256 : per) + 255) / 256 * 256;
  const int n = (a.max_kv_len + per - 1) / per;
  if (n > 1) {
    *chunk = per;
    *n_chunks = n;
  }
}

static int diff_check(const DiffAttnArgs& a, const char* who) {
  NINFER_REQUIRE(a.T > 0 && a.S > 0 && a.Hq > 0 && a.Hkv > 0 && a.dim > 0 && a.vdim > 0 && a.page_size > 0,
                 "%s: sizes must be positive", who);
  NINFER_REQUIRE(a.Hq % a.Hkv == 0, "%s: %d query heads do not split over %d kv heads", who, a.Hq, a.Hkv);
  NINFER_REQUIRE(a.dtype == kF32 || a.dtype == kBF16, "%s: unknown dtype %d", who, a.dtype);
  NINFER_REQUIRE(a.vdim <= 64 * kMaxVPerLane, "%s: value size %d exceeds %d", who, a.vdim, 64 * kMaxVPerLane);
  NINFER_REQUIRE(a.q_stride >= (a.Hq + a.Hkv) * 2 * a.dim + a.Hkv * a.vdim, "%s: rows of %d numbers are too short",
                 who, a.q_stride);
  NINFER_REQUIRE(a.t_coef == 0.f || a.t_every > 0, "%s: the temperature's step must be positive", who);
  NINFER_REQUIRE(a.cap >= 0.f && a.scale > 0.f, "%s: the cap must not be negative, the scale positive", who);
  return 0;
}

}  // namespace ninfer

using namespace ninfer;

extern "C" int ninfer_diff_kv_write(const DiffAttnArgs* a, hipStream_t stream) {
  int rc = diff_check(*a, "diff_kv_write");
  if (rc) return rc;
  if (a->dtype == kF32) diff_kv_write_kernel<float><<<a->T, 256, 0, stream>>>(*a);
  else diff_kv_write_kernel<bf16><<<a->T, 256, 0, stream>>>(*a);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// The single rows at the head of a step that also brings prompt portions, as a step of their
// own (they run as decode rows do); T == 0: there are none, or the kernels for it do not take
// the shape.
static DiffAttnArgs diff_single_rows(const DiffAttnArgs& a) {
  DiffAttnArgs s = a;
  s.T = 0;
  if (a.max_qlen > 1 && a.single_rows > 0 && a.single_rows < a.T && !a.force_plain &&
      diff_attention_tiles_takes(a)) {
    s.T = s.S = a.single_rows;
    s.max_qlen = 1;
    if (!diff_attention_heads_takes(s)) s.T = 0;
  }
  return s;
}

extern "C" long long ninfer_diff_attention_workspace_floats(const DiffAttnArgs* a) {
  int chunk, n;
  const DiffAttnArgs single = diff_single_rows(*a);
  if (single.T > 0) {
    diff_attention_heads_plan(single, &chunk, &n);
    return (long long)single.T * a->Hq * 2 * n * (4 + 2 * a->vdim);
  }
  if (!a->force_plain && diff_attention_heads_takes(*a)) {
    diff_attention_heads_plan(*a, &chunk, &n);
    return (long long)a->T * a->Hq * 2 * n * (4 + 2 * a->vdim);
  }
  diff_chunks(*a, &chunk, &n);
  return n > 1 ? (long long)a->T * a->Hq * n * (4 + 2 * a->vdim) : 0;
}

extern "C" int ninfer_diff_attention(const DiffAttnArgs* a, hipStream_t stream) {
  int rc = diff_check(*a, "diff_attention");
  if (rc) return rc;
  NINFER_REQUIRE(a->out && a->qkv && a->kpool && a->vpool, "diff_attention: null tensors");
  if (a->max_qlen > 1 && !a->force_plain && diff_attention_tiles_takes(*a)) {
    const DiffAttnArgs single = diff_single_rows(*a);
    if (single.T > 0) {
      int chunk, n;
      diff_attention_heads_plan(single, &chunk, &n);
      rc = diff_attention_heads(single, chunk, n, stream);
      if (rc) return rc;
    }
    return diff_attention_tiles(*a, single.T, stream);
  }
  int chunk, n;
  if (!a->force_plain && diff_attention_heads_takes(*a)) {
    diff_attention_heads_plan(*a, &chunk, &n);
    return diff_attention_heads(*a, chunk, n, stream);
  }
  diff_chunks(*a, &chunk, &n);
  if (n > 1)
    NINFER_REQUIRE(a->workspace && a->workspace_floats >= (int64_t)a->T * a->Hq * n * (4 + 2 * a->vdim),
                   "diff_attention: the workspace is too small for %d chunks", n);
  if (diff_rows_takes(*a)) return diff_attention_rows(*a, chunk, n, stream);
  return diff_attention_plain(*a, chunk, n, stream);
}
