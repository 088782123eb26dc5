// Gated linear attention: a recurrent mixer whose state per head is a matrix S [d, dv] with a decay per key
// channel,  S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t,  alpha = sigmoid(z)^(1/tau).
// Each head's o is divided by its root mean square over dv (eps inside the root), multiplied by a weight
// [dv] that the heads share and by silu of a gate row, and written in the activation dtype.
//
// Everything here is 32-bit on both paths: q, k, v, the gate and z arrive as float32 rows of the projections,
// alpha is exp(logsigmoid(z) / tau) with the full-precision functions, the state lives in float32 rows of the
// cache, one per slot, and the norm is 32-bit.
//
// gla_kernel: a block of 256 threads per (sequence, head, CB value columns) walks through the sequence's tokens of
// the step with its part of the state in registers: thread (rg, col) holds RPT neighbouring rows of one column,
// reads them once and writes them once; a single token is the same walk of one step.  The tokens go through LDS
// TC at a time: q, k and the decays of TC tokens are put there by all threads (the next TC tokens' operands are
// already on their way from memory), every thread then updates its rows token by token, with no barrier between
// the tokens, and keeps its TC partial read-outs, which meet in LDS once per TC tokens and are added up in the
// order of the row groups.  CB is 64 where (sequences x heads) fill the chip, else 16, or 8 where even that leaves CUs
// without a block (more blocks, fewer rows a thread).  Which rows belong to the sequence and which state row is its own are read on the device
// (cu_seqlens, slots), so a launch depends on sizes only.  With CB = 64 and dv <= 64 the head's norm and gate are
// finished by the block itself; otherwise o is left in a float32 workspace for gla_finish_kernel (the norm needs
// every column of a head).
#include "common.h"
#include "alice_hip.h"

namespace {

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float silu(float z) { return z / (1.f + expf(-z)); }

// z[t, i] <- sigmoid(z[t, i] + bias[i])^(1 / tau) = exp(logsigmoid(.) / tau), once per key channel for all the blocks
// that share it, with the full-precision functions on both paths.
__global__ void gla_decay_kernel(float* __restrict__ z, const float* __restrict__ bias, float inv_tau, long n, int width) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) z[i] = expf(log_sigmoid(z[i] + bias[i % width]) * inv_tau);
}

template <int CB, int RPT, int TC, typename TW, typename TO>
__global__ __launch_bounds__(256) void gla_kernel(
    const float* __restrict__ rows, int row_w, int q_col, int k_col, int v_col, int g_col,
    const float* __restrict__ alpha, float q_scale, float out_scale,
    const TW* __restrict__ norm_w, float eps, TO* __restrict__ out, float* __restrict__ o32,
    const int* __restrict__ cu_seqlens, const int* __restrict__ slots, float* __restrict__ S, int H, int d, int dv) {
  constexpr int RG = 256 / CB;                 // row groups
  constexpr int DP = RG * RPT;                 // rows the block covers (>= d)
  constexpr int NL = TC * DP / 256;            // q / k / z elements a thread fetches per TC tokens
  constexpr int NV = (TC * CB + 255) / 256;    // v elements, and read-outs, a thread handles per TC tokens
  static_assert(RPT % 4 == 0 && (TC * DP) % 256 == 0, "rows are read four at a time");
  __shared__ __align__(16) float sq[TC][DP];
  __shared__ __align__(16) float sk[TC][DP];
  __shared__ __align__(16) float sa[TC][DP];
  __shared__ float sv[TC][CB];
  __shared__ float red[TC][RG][CB];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, col = tid % CB, rg = tid / CB;
  const int j = blockIdx.z * CB + col;
  const bool col_ok = j < dv;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  if (t1 <= t0) return;
  float* Sh = S + ((size_t)slots[s] * H + h) * d * dv;
  float st[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg * RPT + i;
    st[i] = (r < d && col_ok) ? Sh[(size_t)r * dv + j] : 0.f;
  }
  const bool finish_here = CB == 64 && gridDim.z == 1;
  // what this thread fetches for TC tokens: element (t, r) = (idx / DP, idx % DP) of q, k and the decay; (t, c) of v
  float pq[NL], pk[NL], pz[NL], pv[NV];
  auto fetch = [&](int tc) {
#pragma unroll
    for (int n = 0; n < NL; ++n) {
      const int idx = tid + n * 256, t = tc + idx / DP, r = idx % DP;
      pq[n] = pk[n] = pz[n] = 0.f;
      if (t < t1 && r < d) {
        const float* row = rows + (size_t)t * row_w;
        pq[n] = row[q_col + h * d + r];
        pk[n] = row[k_col + h * d + r];
        pz[n] = alpha[(size_t)t * H * d + h * d + r];
      }
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int idx = tid + n * 256, t = tc + idx / CB, c = blockIdx.z * CB + idx % CB;
      pv[n] = (idx < TC * CB && t < t1 && c < dv) ? rows[(size_t)t * row_w + v_col + h * dv + c] : 0.f;
    }
  };
  fetch(t0);
  for (int tc = t0; tc < t1; tc += TC) {
    const int n_tok = min(TC, t1 - tc);
#pragma unroll
    for (int n = 0; n < NL; ++n) {
      const int idx = tid + n * 256, t = idx / DP, r = idx % DP;
      sq[t][r] = pq[n] * q_scale;
      sk[t][r] = pk[n];
      sa[t][r] = pz[n];                          // (rows beyond d hold zeros and stay zero)
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int idx = tid + n * 256;
      if (idx < TC * CB) sv[idx / CB][idx % CB] = pv[n];
    }
    __syncthreads();
    if (tc + TC < t1) fetch(tc + TC);
    float part[TC];
#pragma unroll
    for (int t = 0; t < TC; ++t) {
      float p = 0.f;
      if (t < n_tok) {
        const float vj = sv[t][col];
#pragma unroll
        for (int i = 0; i < RPT; i += 4) {
          const float4 a = *reinterpret_cast<const float4*>(&sa[t][rg * RPT + i]);
          const float4 kk = *reinterpret_cast<const float4*>(&sk[t][rg * RPT + i]);
          const float4 qq = *reinterpret_cast<const float4*>(&sq[t][rg * RPT + i]);
          st[i] = fmaf(a.x, st[i], kk.x * vj);
          p = fmaf(st[i], qq.x, p);
          st[i + 1] = fmaf(a.y, st[i + 1], kk.y * vj);
          p = fmaf(st[i + 1], qq.y, p);
          st[i + 2] = fmaf(a.z, st[i + 2], kk.z * vj);
          p = fmaf(st[i + 2], qq.z, p);
          st[i + 3] = fmaf(a.w, st[i + 3], kk.w * vj);
          p = fmaf(st[i + 3], qq.w, p);
        }
      }
      part[t] = p;
    }
#pragma unroll
    for (int t = 0; t < TC; ++t) red[t][rg][col] = part[t];
    __syncthreads();
#pragma unroll
    for (int n = 0; n < NV; ++n) {
      const int idx = tid + n * 256, t = idx / CB, c = idx % CB, jj = blockIdx.z * CB + c;
      if (idx >= TC * CB) continue;            // (with CB = 64 a wave has one token: the branch is uniform)
      float o = 0.f;
#pragma unroll
      for (int g = 0; g < RG; ++g) o += red[t][g][c];
      const bool ok = t < n_tok && jj < dv;
      const size_t at = (size_t)(tc + t) * H * dv + h * dv + jj;
      if (finish_here) {
        const float ss = wave_sum(ok ? o * o : 0.f);
        if (ok) {
          const float g = rows[(size_t)(tc + t) * row_w + g_col + h * dv + jj];
          store_f32(out, at, o / sqrtf(ss / (float)dv + eps) * load_f32(norm_w, jj) * silu(g) * out_scale);
        }
      } else if (ok) {
        o32[at] = o;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = rg * RPT + i;
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
// z: float32 [T, H d], the decay's pre-activation without its bias z_bias [H d] (overwritten by the decays); S: [n_slots, H, d, dv] float32;
// out: [T, H dv] in out_dtype, times the constant out_scale; work: float32 [T, H dv] (may be null where (sequences x
// heads) fill the chip and dv <= 64: then nothing is read from it).  columns: value columns a block (0: by the step's size).
extern "C" int alice_gla(const float* rows, int row_w, int q_col, int k_col, int v_col, int g_col, float* z,
                         const float* z_bias, float tau, float q_scale, float out_scale, const void* norm_w, int w_dtype, float eps, void* out,
                         int out_dtype, float* work, const int* cu_seqlens, const int* slots, float* S, int T, int n_seqs,
                         int n_slots, int H, int d, int dv, int columns, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(w_dtype) && dtype_ok(out_dtype), "gla: unknown dtype");
  ALICE_CHECK(columns == 0 || columns == 8 || columns == 16 || columns == 64, "gla: %d value columns a block are not built (8, 16, 64; 0: by the step's size)", columns);
  ALICE_CHECK(rows && z && z_bias && norm_w && out && cu_seqlens && slots && S, "gla: a pointer is missing");
  ALICE_CHECK(T >= 0 && n_seqs >= 0 && n_slots >= 1 && H >= 1 && d >= 1 && dv >= 1, "gla: bad sizes");
  ALICE_CHECK(d <= 256, "gla: key size %d is beyond 256, the range of this kernel", d);
  ALICE_CHECK(tau > 0.f, "gla: tau must be positive");
  ALICE_CHECK(min(min(q_col, k_col), min(v_col, g_col)) >= 0 && max(q_col, k_col) + H * d <= row_w && max(v_col, g_col) + H * dv <= row_w,
              "gla: rows of %d elements are too short for the heads", row_w);
  ALICE_CHECK(H <= 65535 && dv <= 65535 * 16, "gla: too many heads for one launch");
  if (T == 0 || n_seqs == 0) return 0;
  // 64 columns a block where that fills the chip, else 16 (four times the blocks)
  // value columns a block: 64 where that fills the chip twice, else 16, else 8 where 16 leave CUs without a block
  int cb = columns;
  if (cb == 0) cb = (long)n_seqs * H * ceil_div(dv, 64) >= 512 ? 64 : ((long)n_seqs * H * ceil_div(dv, 16) >= 256 ? 16 : 8);
  const bool wide = cb == 64;
  const bool finish_here = wide && dv <= 64;
  ALICE_CHECK(finish_here || work != nullptr, "gla: this shape needs the workspace");
  gla_decay_kernel<<<ceil_div((long)T * H * d, 256), 256, 0, stream>>>(z, z_bias, 1.f / tau, (long)T * H * d, H * d);
  ALICE_LAUNCH_CHECK();
  dim3 grid(n_seqs, H, ceil_div(dv, cb));
#define GO(CB, RPT, TC, TW, TO)                                                                                                  \
  gla_kernel<CB, RPT, TC, TW, TO><<<grid, 256, 0, stream>>>(rows, row_w, q_col, k_col, v_col, g_col, z, q_scale, \
      out_scale, (const TW*)norm_w, eps, (TO*)out, work, cu_seqlens, slots, S, H, d, dv)
#define BY_D(TW, TO)                              \
  do {                                            \
    if (wide) {                                   \
      if (d <= 64) GO(64, 16, 8, TW, TO);         \
      else if (d <= 128) GO(64, 32, 4, TW, TO);   \
      else GO(64, 64, 4, TW, TO);                 \
    } else if (cb == 16) {                        \
      if (d <= 64) GO(16, 4, 16, TW, TO);         \
      else if (d <= 128) GO(16, 8, 16, TW, TO);   \
      else GO(16, 16, 8, TW, TO);                 \
    } else {                                      \
      if (d <= 128) GO(8, 4, 16, TW, TO);         \
      else GO(8, 8, 8, TW, TO);                   \
    }                                             \
  } while (0)
  if (w_dtype == DT_F32 && out_dtype == DT_F32) BY_D(float, float);
  else if (w_dtype == DT_F32) BY_D(float, bf16_t);
  else if (out_dtype == DT_F32) BY_D(bf16_t, float);
  else BY_D(bf16_t, bf16_t);
#undef BY_D
#undef GO
  ALICE_LAUNCH_CHECK();
  if (!finish_here) {
    dim3 g2(T, H);
#define FIN(TW, TO) gla_finish_kernel<TW, TO><<<g2, dv > 128 ? 256 : 64, 0, stream>>>(work, rows, row_w, g_col, (const TW*)norm_w, eps, out_scale, (TO*)out, H, dv)
    if (w_dtype == DT_F32 && out_dtype == DT_F32) FIN(float, float);
    else if (w_dtype == DT_F32) FIN(float, bf16_t);
    else if (out_dtype == DT_F32) FIN(bf16_t, float);
    else FIN(bf16_t, bf16_t);
#undef FIN
    ALICE_LAUNCH_CHECK();
  }
  return 0;
}
