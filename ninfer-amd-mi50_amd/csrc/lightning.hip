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
