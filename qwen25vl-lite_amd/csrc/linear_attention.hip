// Linear attention with a decayed outer-product state, one head at a time:
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t
// S is [LA_DIM, vdim] float32 per (request slot, head).  The decay a_t is one constant per head, or
// one value per key channel and token, a_t = sigmoid(z_t)^(1/tau) from float32 z.  q, k and v are
// columns of the projection's rows (float32 or bfloat16), with an optional silu and a scale on q
// applied in float32 as they are read.  Compiled per key size (-DLA_DIM=...).
//
// The scan: a block of four waves owns 64 value channels of one head of one request and walks the
// request's tokens of this step in order, starting from the state its slot holds and leaving the
// new state there.  Lane = value channel; each wave keeps LA_DIM / 4 rows of S in registers.
// Tokens are staged LA_TB at a time: q, k and the decays go to LDS (every lane reads the same
// word), the four partial sums of o meet in LDS.  The order of every sum is fixed by the sizes
// alone, so a token's result does not depend on how its sequence was cut into steps or on what
// else the batch holds.
//
// One prompt alone has only heads x vdim / 64 such blocks.  With G > 1 the key channels are cut
// into G groups, each with blocks of its own (four waves of LA_DIM / (4 G) rows); a group's sums of
// o go to its own slab of the output, [G, N, heads * vdim], and whoever reads the output adds the
// slabs in order (the norm that follows does).
#include "common.h"

#ifndef LA_DIM
#define LA_DIM 64
#endif
#define LA_WAVES 4
#define LA_TB (LA_DIM > 128 ? 8 : 16)

static_assert(LA_DIM % LA_WAVES == 0, "the key size must be a multiple of 4");

__device__ __forceinline__ float la_act(float z, int act) { return act ? z / (1.0f + expf(-z)) : z; }

// log(sigmoid(z)) = min(z, 0) - log1p(exp(-|z|))
__device__ __forceinline__ float la_decay(float z, float inv_tau) {
  return expf((fminf(z, 0.f) - log1pf(expf(-fabsf(z)))) * inv_tau);
}

template <typename TP, bool CHANNEL_DECAY, int G>
__global__ __launch_bounds__(256) void la_scan_kernel(
    const TP* __restrict__ proj, long long proj_stride, int q_off, int k_off, int v_off,
    const float* __restrict__ head_decay, const float* __restrict__ z, long long z_stride, float inv_tau,
    float* __restrict__ state, const int* __restrict__ cu_q, const int* __restrict__ req_slots,
    float* __restrict__ out, long long out_slab, int H, int vdim, int act, float q_scale) {
  // key channels of this block's group (a G that does not divide the rows among the waves is never launched)
  constexpr int DG = LA_DIM % (LA_WAVES * G) == 0 ? LA_DIM / G : LA_DIM;
  constexpr int LA_ROWS = DG / LA_WAVES;    // rows of S a wave keeps
  __shared__ float qs[LA_TB][DG];
  __shared__ float ks[LA_TB][DG];
  __shared__ float as[CHANNEL_DECAY ? LA_TB : 1][DG];
  __shared__ float po[LA_TB][LA_WAVES][64];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int head = blockIdx.y, req = blockIdx.z;
  const int vtile = blockIdx.x / G, group = blockIdx.x % G;
  const int d0 = group * DG;
  const int vcol = vtile * 64 + lane;
  const bool live = vcol < vdim;
  const int begin = cu_q[req], end = cu_q[req + 1];
  if (begin >= end) return;
  out += (size_t)group * out_slab;
  float* srow = state + (((size_t)req_slots[req] * H + head) * LA_DIM + d0 + (size_t)wave * LA_ROWS) * vdim + vcol;
  float S[LA_ROWS];
#pragma unroll
  for (int i = 0; i < LA_ROWS; ++i) S[i] = live ? srow[(size_t)i * vdim] : 0.f;
  const float fixed = CHANNEL_DECAY ? 1.f : head_decay[head];

  for (int t0 = begin; t0 < end; t0 += LA_TB) {
    const int nt = end - t0 < LA_TB ? end - t0 : LA_TB;
    for (int idx = tid; idx < nt * DG; idx += 256) {
      const int t = idx / DG, d = idx % DG;
      const TP* row = proj + (size_t)(t0 + t) * proj_stride + (size_t)head * LA_DIM + d0 + d;
      qs[t][d] = la_act(ldf<TP>(row + q_off), act) * q_scale;
      ks[t][d] = la_act(ldf<TP>(row + k_off), act);
      if (CHANNEL_DECAY)
        as[t][d] = la_decay(z[(size_t)(t0 + t) * z_stride + (size_t)head * LA_DIM + d0 + d], inv_tau);
    }
    float vt[LA_TB];
#pragma unroll
    for (int t = 0; t < LA_TB; ++t)
      vt[t] = (live && t < nt)
                  ? la_act(ldf<TP>(proj + (size_t)(t0 + t) * proj_stride + v_off + (size_t)head * vdim + vcol), act)
                  : 0.f;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < LA_TB; ++t) {
      if (t < nt) {
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < LA_ROWS; ++i) {
          const int d = wave * LA_ROWS + i;
          const float a = CHANNEL_DECAY ? as[t][d] : fixed;
          S[i] = a * S[i] + ks[t][d] * vt[t];
          acc += S[i] * qs[t][d];
        }
        po[t][wave][lane] = acc;
      }
    }
    __syncthreads();
    for (int idx = tid; idx < nt * 64; idx += 256) {
      const int t = idx >> 6, l = idx & 63;
      const int c = vtile * 64 + l;
      if (c < vdim)
        out[((size_t)(t0 + t) * H + head) * vdim + c] = ((po[t][0][l] + po[t][1][l]) + po[t][2][l]) + po[t][3][l];
    }
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < LA_ROWS; ++i) srow[(size_t)i * vdim] = S[i];
  }
}

extern "C" int qvl_la_key_size() { return LA_DIM; }

// proj: rows of `proj_stride` values holding q (H * LA_DIM columns from q_off), k (from k_off) and v
// (H * vdim columns from v_off).  head_decay [H] float32, or z float32 rows (H * LA_DIM columns) with
// inv_tau.  state [slots, H, LA_DIM, vdim] float32; cu_q [R + 1], req_slots [R]; out float32
// [groups, N, H * vdim] (groups 1, 2, 4 or 8 with LA_DIM a multiple of 4 * groups), slabs `out_slab` apart.
extern "C" int qvl_la_scan(const void* proj, long long proj_stride, int q_off, int k_off, int v_off, int proj_dtype,
                           const void* head_decay, const void* z, long long z_stride, float inv_tau, void* state,
                           const void* cu_q, const void* req_slots, void* out, long long out_slab, int groups, int R,
                           int H, int dim, int vdim, int act, float q_scale, hipStream_t stream) {
  if (R <= 0) return QVL_OK;
  if (dim != LA_DIM || H <= 0 || vdim <= 0 || (!head_decay && !z)) return QVL_ERR_SHAPE;
  if (groups != 1 && groups != 2 && groups != 4 && groups != 8) return QVL_ERR_SHAPE;
  if (LA_DIM % (LA_WAVES * groups)) return QVL_ERR_SHAPE;
  if (H > 65535 || R > 65535) return QVL_ERR_LIMIT;
  const dim3 grid(((vdim + 63) / 64) * groups, H, R);
#define LAUNCH(TP, CH, G)                                                                                           \
  hipLaunchKernelGGL((la_scan_kernel<TP, CH, G>), grid, dim3(256), 0, stream, (const TP*)proj, proj_stride, q_off,   \
                     k_off, v_off, (const float*)head_decay, (const float*)z, z_stride, inv_tau, (float*)state,      \
                     (const int*)cu_q, (const int*)req_slots, (float*)out, out_slab, H, vdim, act, q_scale)
#define BY_GROUPS(TP, CH)                                                                                           \
  switch (groups) {                                                                                                 \
    case 1: LAUNCH(TP, CH, 1); break;                                                                               \
    case 2: LAUNCH(TP, CH, 2); break;                                                                               \
    case 4: LAUNCH(TP, CH, 4); break;                                                                               \
    default: LAUNCH(TP, CH, 8); break;                                                                              \
  }
  if (proj_dtype == 0) { if (z) { BY_GROUPS(float, true) } else { BY_GROUPS(float, false) } }
  else if (proj_dtype == 1) { if (z) { BY_GROUPS(bf16_t, true) } else { BY_GROUPS(bf16_t, false) } }
  else return QVL_ERR_DTYPE;
#undef BY_GROUPS
#undef LAUNCH
  return qvl_launch_status();
}
