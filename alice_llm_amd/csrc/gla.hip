// Gated linear attention: a recurrent mixer whose state per head is a matrix S [d, dv] with a decay per key
// channel,  S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t,  alpha = sigmoid(z)^(1/tau).
// Each head's o is divided by its root mean square over dv (eps inside the root), multiplied by a weight
// [dv] that the heads share and by silu of a gate row, and written in the activation dtype.
//
// Everything here is 32-bit on both paths: q, k, v, the gate and z arrive as float32 rows of the projections,
// alpha is exp(logsigmoid(z) / tau) with the full-precision functions, the state lives in float32 rows of the
// cache, one per slot, and the norm is 32-bit.
//
// gla_kernel: a block of four waves per (sequence, head, 64 value columns) walks through the sequence's tokens
// of the step with its part of the state in registers (thread (rg, lane) holds rows rg, rg + 4, ... of column
// lane), reads the state once and writes it once; a single token is the same walk of one step.  The next
// token's operands are fetched while the current one is worked on.  Which rows belong to the sequence and
// which state row is its own are read on the device (cu_seqlens, slots), so a launch depends on sizes only.
// With dv <= 64 the head's norm and gate are finished by the block itself; wider heads leave o in a float32
// workspace for gla_finish_kernel (the norm needs every column of a head).
#include "common.h"
#include "alice_hip.h"

namespace {

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float silu(float z) { return z / (1.f + expf(-z)); }

template <int RPT, typename TW, typename TO>
__global__ __launch_bounds__(256) void gla_kernel(
    const float* __restrict__ rows, int row_w, int q_col, int k_col, int v_col, int g_col,
    const float* __restrict__ z, const float* __restrict__ z_bias, float inv_tau, float q_scale, float out_scale,
    const TW* __restrict__ norm_w, float eps, TO* __restrict__ out, float* __restrict__ o32,
    const int* __restrict__ cu_seqlens, const int* __restrict__ slots, float* __restrict__ S, int H, int d, int dv) {
  __shared__ float sq[256], sk[256], sa[256];
  __shared__ float red[4][64];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, rg = tid >> 6;
  const int j = blockIdx.z * 64 + lane;
  const bool col_ok = j < dv;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  if (t1 <= t0) return;
  float* Sh = S + ((size_t)slots[s] * H + h) * d * dv;
  float st[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg + 4 * i;
    st[i] = (r < d && col_ok) ? Sh[(size_t)r * dv + j] : 0.f;
  }
  const bool finish_here = gridDim.z == 1;
  // this thread's operands of the token: element tid of q, k and z (tid < d), element j of v
  float nq = 0.f, nk = 0.f, nz = 0.f, nv = 0.f;
  auto fetch = [&](int t) {
    const float* row = rows + (size_t)t * row_w;
    if (tid < d) {
      nq = row[q_col + h * d + tid];
      nk = row[k_col + h * d + tid];
      nz = z[(size_t)t * H * d + h * d + tid];
    }
    if (col_ok) nv = row[v_col + h * dv + j];
  };
  fetch(t0);
  for (int t = t0; t < t1; ++t) {
    if (tid < d) {
      sq[tid] = nq * q_scale;
      sk[tid] = nk;
      sa[tid] = expf(log_sigmoid(nz + z_bias[h * d + tid]) * inv_tau);
    }
    const float vj = nv;
    __syncthreads();
    if (t + 1 < t1) fetch(t + 1);
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int r = rg + 4 * i;
      if (r < d) {
        st[i] = fmaf(sa[r], st[i], sk[r] * vj);
        part = fmaf(st[i], sq[r], part);
      }
    }
    red[rg][lane] = part;
    __syncthreads();
    if (rg == 0) {
      const float o = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
      if (finish_here) {
        const float ss = wave_sum(col_ok ? o * o : 0.f);
        if (col_ok) {
          const float g = rows[(size_t)t * row_w + g_col + h * dv + j];
          const float y = o / sqrtf(ss / (float)dv + eps) * load_f32(norm_w, j) * silu(g) * out_scale;
          store_f32(out + (size_t)t * H * dv + h * dv, j, y);
        }
      } else if (col_ok) {
        o32[(size_t)t * H * dv + h * dv + j] = o;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg + 4 * i;
    if (r < d && col_ok) Sh[(size_t)r * dv + j] = st[i];
  }
}

// The head norm, its weight and the gate for heads wider than one block's columns: a block per (token, head).
template <typename TW, typename TO>
__global__ __launch_bounds__(256) void gla_finish_kernel(const float* __restrict__ o32, const float* __restrict__ rows, int row_w,
                                                         int g_col, const TW* __restrict__ norm_w, float eps, float out_scale,
                                                         TO* __restrict__ out, int H, int dv) {
  __shared__ float red[17];
  const int t = blockIdx.x, h = blockIdx.y;
  const float* o = o32 + ((size_t)t * H + h) * dv;
  float ss = 0.f;
  for (int e = threadIdx.x; e < dv; e += blockDim.x) ss = fmaf(o[e], o[e], ss);
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)dv + eps);
  for (int e = threadIdx.x; e < dv; e += blockDim.x) {
    const float g = rows[(size_t)t * row_w + g_col + h * dv + e];
    store_f32(out + ((size_t)t * H + h) * dv, e, o[e] * inv * load_f32(norm_w, e) * silu(g) * out_scale);
  }
}

}  // namespace

// rows: float32 [T, row_w] with q at q_col (H d), k at k_col (H d), v at v_col (H dv) and the gate at g_col (H dv);
// z: float32 [T, H d], the decay's pre-activation without its bias z_bias [H d]; S: [n_slots, H, d, dv] float32;
// out: [T, H dv] in out_dtype, times the constant out_scale; work: float32 [T, H dv], read only where dv > 64.
extern "C" int alice_gla(const float* rows, int row_w, int q_col, int k_col, int v_col, int g_col, const float* z,
                         const float* z_bias, float tau, float q_scale, float out_scale, const void* norm_w, int w_dtype, float eps, void* out,
                         int out_dtype, float* work, const int* cu_seqlens, const int* slots, float* S, int T, int n_seqs,
                         int n_slots, int H, int d, int dv, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(w_dtype) && dtype_ok(out_dtype), "gla: unknown dtype");
  ALICE_CHECK(rows && z && z_bias && norm_w && out && cu_seqlens && slots && S, "gla: a pointer is missing");
  ALICE_CHECK(T >= 0 && n_seqs >= 0 && n_slots >= 1 && H >= 1 && d >= 1 && dv >= 1, "gla: bad sizes");
  ALICE_CHECK(d <= 256, "gla: key size %d is beyond 256, the range of this kernel", d);
  ALICE_CHECK(dv <= 64 || work != nullptr, "gla: value heads wider than 64 need the workspace");
  ALICE_CHECK(tau > 0.f, "gla: tau must be positive");
  ALICE_CHECK(min(min(q_col, k_col), min(v_col, g_col)) >= 0 && max(q_col, k_col) + H * d <= row_w && max(v_col, g_col) + H * dv <= row_w,
              "gla: rows of %d elements are too short for the heads", row_w);
  ALICE_CHECK(H <= 65535 && ceil_div(dv, 64) <= 65535, "gla: too many heads for one launch");
  if (T == 0 || n_seqs == 0) return 0;
  dim3 grid(n_seqs, H, ceil_div(dv, 64));
#define GO(RPT, TW, TO)                                                                                                         \
  gla_kernel<RPT, TW, TO><<<grid, 256, 0, stream>>>(rows, row_w, q_col, k_col, v_col, g_col, z, z_bias, 1.f / tau, q_scale, out_scale, \
      (const TW*)norm_w, eps, (TO*)out, work, cu_seqlens, slots, S, H, d, dv)
#define BY_D(TW, TO)                 \
  do {                               \
    if (d <= 64) GO(16, TW, TO);     \
    else if (d <= 128) GO(32, TW, TO); \
    else GO(64, TW, TO);             \
  } while (0)
  if (w_dtype == DT_F32 && out_dtype == DT_F32) BY_D(float, float);
  else if (w_dtype == DT_F32) BY_D(float, bf16_t);
  else if (out_dtype == DT_F32) BY_D(bf16_t, float);
  else BY_D(bf16_t, bf16_t);
#undef BY_D
#undef GO
  ALICE_LAUNCH_CHECK();
  if (dv > 64) {
    dim3 g2(T, H);
#define FIN(TW, TO) gla_finish_kernel<TW, TO><<<g2, 256, 0, stream>>>(work, rows, row_w, g_col, (const TW*)norm_w, eps, out_scale, (TO*)out, H, dv)
    if (w_dtype == DT_F32 && out_dtype == DT_F32) FIN(float, float);
    else if (w_dtype == DT_F32) FIN(float, bf16_t);
    else if (out_dtype == DT_F32) FIN(bf16_t, float);
    else FIN(bf16_t, bf16_t);
#undef FIN
    ALICE_LAUNCH_CHECK();
  }
  return 0;
}
