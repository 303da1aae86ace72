// Linear attention with a per-head decay ("lightning attention"), token by token:
//
//   S_t = decay_h S_(t-1) + k_t v_t^T      (S: [dim, vdim] per head, 32-bit, per-request state)
//   o_t = S_t^T q_t
//
// q, k, v are silu of the projected rows (the activation is applied here, in 32-bit, to the
// projection's stored value). One block per (request, head) walks the request's rows of the
// step in order; the state comes from and returns to the request's slot, so a request may be
// cut into steps anywhere and every row sees exactly the sums it would see in one piece.
// Thread (part, v) owns S[d][v] for d = part, part + parts, ...: it updates them and forms its
// part of o_t[v] in the same pass; the parts are added in ascending order. The order of
// every sum depends on (dim, vdim) alone.
#include "common.h"

namespace ninfer {

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }

template <typename T>
__global__ void lightning_seq_kernel(const T* __restrict__ qkv, int stride, int q_off, int k_off,
                                     int v_off, const float* __restrict__ decay,
                                     float* __restrict__ state, int64_t state_stride,
                                     float* __restrict__ out, const int* __restrict__ seq_row_start,
                                     const int* __restrict__ seq_slots, int H, int dim, int vdim,
                                     int parts) {
  extern __shared__ float smem[];
  float* S = smem;                       // [dim * vdim]
  float* qk = S + dim * vdim;            // 2 x [2 dim + vdim]: q, k, v of a row, two buffers
  float* part_s = qk + 2 * (2 * dim + vdim);   // [parts * vdim]
  const int s = blockIdx.x, h = blockIdx.y;
  const int r0 = seq_row_start[s], n = seq_row_start[s + 1] - r0;
  float* st = state + (int64_t)seq_slots[s] * state_stride + (int64_t)h * dim * vdim;
  const int tid = threadIdx.x;
  const int vv = tid % vdim, part = tid / vdim;   // blockDim.x == parts * vdim
  for (int e = tid; e < dim * vdim; e += blockDim.x) S[e] = st[e];
  const float dec = decay[h];
  const int row_floats = 2 * dim + vdim;
  for (int i = 0; i < n; ++i) {
    float* buf = qk + (i & 1) * row_floats;
    const T* row = qkv + (int64_t)(r0 + i) * stride;
    for (int e = tid; e < row_floats; e += blockDim.x) {
      int col = e < dim ? q_off + h * dim + e
                        : e < 2 * dim ? k_off + h * dim + (e - dim) : v_off + h * vdim + (e - 2 * dim);
      buf[e] = silu_f(to_f32(row[col]));
    }
    __syncthreads();   // the row is in LDS; the state of the previous row is complete
    const float* q_s = buf;
    const float* k_s = buf + dim;
    const float v_t = buf[2 * dim + vv];
    float acc = 0.f;
    for (int d = part; d < dim; d += parts) {
      const float sn = fmaf(dec, S[d * vdim + vv], k_s[d] * v_t);
      S[d * vdim + vv] = sn;
      acc = fmaf(sn, q_s[d], acc);
    }
    part_s[part * vdim + vv] = acc;
    __syncthreads();
    if (part == 0) {
      float o = 0.f;
      for (int p = 0; p < parts; ++p) o += part_s[p * vdim + vv];
      out[((int64_t)(r0 + i) * H + h) * vdim + vv] = o;
    }
    // the next row writes the other q/k/v buffer, and part_s only after its first barrier
  }
  __syncthreads();
  for (int e = tid; e < dim * vdim; e += blockDim.x) st[e] = S[e];
}

}  // namespace ninfer

using namespace ninfer;

// qkv: [T, stride] rows of the activation dtype with the heads' q at column q_off, k at
// k_off (heads x dim each) and v at v_off (heads x vdim); out: [T, heads * vdim] 32-bit.
extern "C" int ninfer_lightning_attention(const void* qkv, int stride, int q_off, int k_off,
                                          int v_off, const float* decay, float* state,
                                          long long state_stride, float* out,
                                          const int* seq_row_start, const int* seq_slots, int T,
                                          int S, int H, int dim, int vdim, int dtype,
                                          hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && S > 0 && H > 0 && dim > 0 && vdim > 0,
                 "lightning_attention: T=%d S=%d heads=%d dim=%d vdim=%d must be positive", T, S,
                 H, dim, vdim);
  NINFER_REQUIRE(vdim <= 1024, "lightning_attention: value size %d exceeds 1024", vdim);
  NINFER_REQUIRE(state_stride >= (long long)H * dim * vdim,
                 "lightning_attention: a request's state of %lld floats holds no %d x %d x %d",
                 state_stride, H, dim, vdim);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "lightning_attention: unknown dtype %d", dtype);
  int parts = 256 / vdim;
  if (parts < 1) parts = 1;
  if (parts > dim) parts = dim;
  const int block = parts * vdim;
  const size_t lds = ((size_t)dim * vdim + 2 * (2 * dim + vdim) + (size_t)parts * vdim) * sizeof(float);
  NINFER_REQUIRE(lds <= 160 * 1024, "lightning_attention: a head's state of %d x %d does not fit "
                 "the LDS", dim, vdim);
  const dim3 grid(S, H);
#define NINFER_LIGHTNING_LAUNCH(TYPE)                                                          \
  do {                                                                                         \
    auto kern = lightning_seq_kernel<TYPE>;                                                    \
    if (lds > 48 * 1024) {                                                                     \
      hipError_t e = hipFuncSetAttribute((const void*)kern,                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) return set_error(-2, "lightning_attention: cannot get %zu bytes of LDS", lds); \
    }                                                                                          \
    kern<<<grid, block, lds, stream>>>((const TYPE*)qkv, stride, q_off, k_off, v_off, decay,   \
                                       state, state_stride, out, seq_row_start, seq_slots, H,  \
                                       dim, vdim, parts);                                      \
  } while (0)
  if (dtype == kF32)
    NINFER_LIGHTNING_LAUNCH(float);
  else
    NINFER_LIGHTNING_LAUNCH(bf16);
#undef NINFER_LIGHTNING_LAUNCH
  NINFER_LAUNCH_CHECK();
  return 0;
}

// ---- prompt portions in chunks, on the 32-bit matrix instruction --------------------------------
//
// For the rows i = 0 .. L - 1 of a chunk (L <= 64) with the state S before it:
//
//   o_i = sum_{j <= i} d^(i - j) (q_i . k_j) v_j  +  d^(i + 1) S^T q_i
//   S' = d^L S + sum_j d^(L - 1 - j) k_j v_j^T
//
// which is the recurrence written out; all powers of the decay have exponents >= 0, so nothing
// grows. Every product runs on v_mfma_f32_32x32x2_f32: q, k, v (silu of the projections), the
// decays and the state enter in 32-bit and are never rounded to a shorter type. A block owns
// one (request, head, 32 value columns): the chunks of a request follow each other in it, and
// the value columns of a head are independent, which gives the launch heads x vdim / 32 blocks
// per request. Waves 0 and 1 form the chunk's outputs, waves 2 and 3 carry the state in their
// accumulators and hand a copy to the others through LDS.
namespace ninfer {

typedef float lt_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 lt_bf16x8 __attribute__((ext_vector_type(8)));
constexpr int kLtChunk = 64;
constexpr int kLtStateTiles = 4;   // 32-row tiles of the state per carrying wave: dim up to 256

__device__ __forceinline__ float decay_pow(float log2d, int n) {
  return n == 0 ? 1.f : exp2f((float)n * log2d);   // (a decay of 0 has log2 -inf: 0 * -inf is no number)
}

template <typename T>
__global__ __launch_bounds__(256) void lightning_chunk_kernel(
    const T* __restrict__ qkv, int stride, int q_off, int k_off, int v_off,
    const float* __restrict__ decay, float* __restrict__ state, int64_t state_stride,
    float* __restrict__ out, const int* __restrict__ seq_row_start,
    const int* __restrict__ seq_slots, int H, int dim, int vdim) {
  extern __shared__ float smem[];
  const int qs = dim + 1;                 // row length of q and k in LDS (odd: column reads spread)
  float* Qs = smem;                       // [64][dim + 1]
  float* Ks = Qs + kLtChunk * qs;         // [64][dim + 1]
  float* Vs = Ks + kLtChunk * qs;         // [64][33]
  float* As = Vs + kLtChunk * 33;         // [64][65]
  float* Ss = As + kLtChunk * 65;         // [dim32][33]
  float* Ws = Ss + ((dim + 31) / 32 * 32) * 33;   // [64] d^(L - 1 - j) of the chunk's rows
  const int s = blockIdx.x, h = blockIdx.y, c0 = 32 * blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, lr = lane & 31, lk = lane >> 5;
  const int r0 = seq_row_start[s], n = seq_row_start[s + 1] - r0;
  const int dim32 = (dim + 31) / 32 * 32;
  const int d_tiles = dim32 / 32;
  float* st = state + (int64_t)seq_slots[s] * state_stride + (int64_t)h * dim * vdim;
  const float dec = decay[h];
  const float log2d = log2f(dec);
  const bool col_ok = c0 + lr < vdim;
  // rows of bfloat16 whose q and k parts start at multiples of 16 bytes
  const bool wide = sizeof(T) == 2 && dim % 8 == 0 && stride % 8 == 0 && q_off % 8 == 0 &&
                    k_off % 8 == 0 && ((uintptr_t)qkv % 16 == 0);

  // the state: in the accumulators of waves 2 and 3 (tiles w - 2, w, ...), a copy in LDS
  lt_f32x16 sacc[kLtStateTiles];
#pragma unroll
  for (int x = 0; x < kLtStateTiles; ++x)
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[x][i] = 0.f;
  for (int e = tid; e < dim32 * 33; e += 256) {
    const int d = e / 33, c = e % 33;
    Ss[e] = (d < dim && c < 32 && c0 + c < vdim) ? st[(int64_t)d * vdim + c0 + c] : 0.f;
  }
  __syncthreads();
  if (w >= 2) {
#pragma unroll
    for (int x = 0; x < kLtStateTiles; ++x) {
      const int dt = (w - 2) + 2 * x;
      if (dt < d_tiles) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) sacc[x][4 * q + r] = Ss[(32 * dt + 8 * q + 4 * lk + r) * 33 + lr];
      }
    }
  }

  for (int i0 = 0; i0 < n; i0 += kLtChunk) {
    const int L = min(kLtChunk, n - i0);
    // 1. the chunk's q, k (all of the head's numbers) and this block's value columns
    if (wide) {   // eight neighbouring numbers per load
      const int per_row = dim / 8;
      for (int e = tid; e < kLtChunk * per_row; e += 256) {
        const int i = e / per_row, d = 8 * (e % per_row);
        float qv[8], kv[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) qv[x] = kv[x] = 0.f;
        if (i < L) {
          const T* row = qkv + (int64_t)(r0 + i0 + i) * stride;
          const lt_bf16x8 a = *(const lt_bf16x8*)(row + q_off + h * dim + d);
          const lt_bf16x8 b = *(const lt_bf16x8*)(row + k_off + h * dim + d);
#pragma unroll
          for (int x = 0; x < 8; ++x) {
            qv[x] = silu_f((float)a[x]);
            kv[x] = silu_f((float)b[x]);
          }
        }
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          Qs[i * qs + d + x] = qv[x];
          Ks[i * qs + d + x] = kv[x];
        }
      }
    } else {
      for (int e = tid; e < kLtChunk * dim; e += 256) {
        const int i = e / dim, d = e % dim;
        float qv = 0.f, kv = 0.f;
        if (i < L) {
          const T* row = qkv + (int64_t)(r0 + i0 + i) * stride;
          qv = silu_f(to_f32(row[q_off + h * dim + d]));
          kv = silu_f(to_f32(row[k_off + h * dim + d]));
        }
        Qs[i * qs + d] = qv;
        Ks[i * qs + d] = kv;
      }
    }
    for (int e = tid; e < kLtChunk * 32; e += 256) {
      const int i = e >> 5, c = e & 31;
      float vv = 0.f;
      if (i < L && c0 + c < vdim)
        vv = silu_f(to_f32(qkv[(int64_t)(r0 + i0 + i) * stride + v_off + h * vdim + c0 + c]));
      Vs[i * 33 + c] = vv;
    }
    if (tid < kLtChunk) Ws[tid] = tid < L ? decay_pow(log2d, L - 1 - tid) : 0.f;
    __syncthreads();   // (also: the state's copy in LDS is the one before this chunk)
    // 2. A[i][j] = d^(i - j) q_i . k_j for j <= i: wave w has rows 32 (w / 2).., keys 32 (w % 2)..
    {
      const int mi = w >> 1, nj = w & 1;
      lt_f32x16 a;
#pragma unroll
      for (int i = 0; i < 16; ++i) a[i] = 0.f;
      if (nj <= mi) {
        const float* qrow = Qs + (32 * mi + lr) * qs + lk;
        const float* krow = Ks + (32 * nj + lr) * qs + lk;
#pragma unroll 8
        for (int d = 0; d < dim; d += 2) {
          const float qa = (d + lk < dim) ? qrow[d] : 0.f;
          const float kb = (d + lk < dim) ? krow[d] : 0.f;
          a = __builtin_amdgcn_mfma_f32_32x32x2f32(qa, kb, a, 0, 0, 0);
        }
      }
      const int j = 32 * nj + lr;
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = 32 * mi + 8 * q + 4 * lk + r;
          As[i * 65 + j] = j <= i ? a[4 * q + r] * decay_pow(log2d, i - j) : 0.f;
        }
    }
    __syncthreads();
    // 3. waves 0, 1: the outputs of rows 32 w ..; waves 2, 3: the state after the chunk
    if (w < 2) {
      lt_f32x16 o;
#pragma unroll
      for (int i = 0; i < 16; ++i) o[i] = 0.f;
      const int row = 32 * w + lr;
      const float* arow = As + row * 65 + lk;
#pragma unroll 8
      for (int j = 0; j < 32 * (w + 1); j += 2)
        o = __builtin_amdgcn_mfma_f32_32x32x2f32(arow[j], Vs[(j + lk) * 33 + lr], o, 0, 0, 0);
      const float carry = decay_pow(log2d, row + 1);
      const float* qrow = Qs + row * qs + lk;
#pragma unroll 8
      for (int d = 0; d < dim; d += 2) {
        const float qa = (d + lk < dim) ? qrow[d] * carry : 0.f;
        o = __builtin_amdgcn_mfma_f32_32x32x2f32(qa, Ss[(d + lk) * 33 + lr], o, 0, 0, 0);
      }
      if (col_ok) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int i = 32 * w + 8 * q + 4 * lk + r;
            if (i < L) out[((int64_t)(r0 + i0 + i) * H + h) * vdim + c0 + lr] = o[4 * q + r];
          }
      }
    } else {
      const float whole = decay_pow(log2d, L);
#pragma unroll
      for (int x = 0; x < kLtStateTiles; ++x) {
        const int dt = (w - 2) + 2 * x;
        if (dt < d_tiles) {
#pragma unroll
          for (int i = 0; i < 16; ++i) sacc[x][i] *= whole;
          const int d = 32 * dt + lr;
#pragma unroll 8
          for (int j = 0; j < kLtChunk; j += 2) {
            const int jj = j + lk;
            const float ka = (jj < L && d < dim) ? Ks[jj * qs + d] * Ws[jj] : 0.f;
            sacc[x] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka, Vs[jj * 33 + lr], sacc[x], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();   // everyone has read the old copy of the state
    if (w >= 2) {
#pragma unroll
      for (int x = 0; x < kLtStateTiles; ++x) {
        const int dt = (w - 2) + 2 * x;
        if (dt < d_tiles) {
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int r = 0; r < 4; ++r) Ss[(32 * dt + 8 * q + 4 * lk + r) * 33 + lr] = sacc[x][4 * q + r];
        }
      }
    }
    // (the barrier after the next chunk's loads publishes the copy; nothing reads it before)
  }
  if (w >= 2 && col_ok) {
#pragma unroll
    for (int x = 0; x < kLtStateTiles; ++x) {
      const int dt = (w - 2) + 2 * x;
      if (dt < d_tiles) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int d = 32 * dt + 8 * q + 4 * lk + r;
            if (d < dim) st[(int64_t)d * vdim + c0 + lr] = sacc[x][4 * q + r];
          }
      }
    }
  }
}

static size_t lightning_chunk_lds(int dim) {
  const int dim32 = (dim + 31) / 32 * 32;
  return ((size_t)2 * kLtChunk * (dim + 1) + kLtChunk * 33 + kLtChunk * 65 + (size_t)dim32 * 33 + kLtChunk) * sizeof(float);
}

}  // namespace ninfer

// The same as ninfer_lightning_attention for bfloat16 rows, chunk by chunk on the matrix cores:
// for steps that bring prompt portions. Returns 1 (nothing launched) when the sizes do not fit.
extern "C" int ninfer_lightning_attention_chunks(const void* qkv, int stride, int q_off, int k_off,
                                                 int v_off, const float* decay, float* state,
                                                 long long state_stride, float* out,
                                                 const int* seq_row_start, const int* seq_slots,
                                                 int T, int S, int H, int dim, int vdim, int dtype,
                                                 hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && S > 0 && H > 0 && dim > 0 && vdim > 0,
                 "lightning_attention: T=%d S=%d heads=%d dim=%d vdim=%d must be positive", T, S,
                 H, dim, vdim);
  NINFER_REQUIRE(state_stride >= (long long)H * dim * vdim,
                 "lightning_attention: a request's state of %lld floats holds no %d x %d x %d",
                 state_stride, H, dim, vdim);
  const size_t lds = lightning_chunk_lds(dim);
  if (dtype != kBF16 || dim > 64 * kLtStateTiles || lds > 160 * 1024) return 1;
  auto kern = lightning_chunk_kernel<bf16>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds);
    if (e != hipSuccess) return set_error(-2, "lightning_attention: cannot get %zu bytes of LDS", lds);
  }
  kern<<<dim3(S, H, (vdim + 31) / 32), 256, lds, stream>>>(
      (const bf16*)qkv, stride, q_off, k_off, v_off, decay, state, state_stride, out,
      seq_row_start, seq_slots, H, dim, vdim);
  NINFER_LAUNCH_CHECK();
  return 0;
}
