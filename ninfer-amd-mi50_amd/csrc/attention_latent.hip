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
// The rotation turns pair (i, i + n/2) of the first n = rot_n numbers of the rotated part by
// pos * freq[i]; cosine and sine are multiplied by `magnitude` (1 without a scaled table).
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
        const int p = i < half ? i : i - half;
        float x, y;
        turn_pair(to_f32(kr[p]), to_f32(kr[p + half]), trig[p], trig[half + p], &x, &y);
        v = i < half ? x : y;
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
      const int p = i < half ? i : i - half;
      float x, y;
      turn_pair(to_f32(qr[p]), to_f32(qr[p + half]), trig[p], trig[half + p], &x, &y);
      v = i < half ? x : y;
    }
    a.q_abs[((int64_t)t * a.Hq + h) * Dk + a.R + i] = v;
  }
}

constexpr int kLatentMaxPerLane = 8;   // latent sizes up to 512

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
