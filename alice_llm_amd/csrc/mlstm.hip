// The matrix memory (mLSTM): per sequence and head a matrix S [d, dv], a vector n [d] and a stabiliser m,
// all 32-bit and carried from token to token in the cache's state tensors.
//
// For token t of a head, with the raw gate numbers a = W_i h + b_i and b = W_f h + b_f:
//   i  = cap * tanh(a / cap)                      log input gate
//   f  = logsigmoid(cap * tanh(b / cap))          log forget gate
//   m' = max(f + m, i)
//   S' = exp(f + m - m') S + exp(i - m') k v^T,   n' likewise with k alone
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6),  q scaled by d^(-1/2)
// and, fused behind it, what the mixer does with o before its output matrix: o divided by its root mean
// square over the head (eps inside the root), times the norm weight, times sigmoid of the output gate.
// m starts at 0 (the state tensors are zero when a sequence starts), which is the design's choice; with
// `cap` <= 0 the gates are used uncapped.
//
// Everything here is 32-bit with full-precision exp/tanh/log on every path; only the result is written in
// the activation dtype.  The rows come from the fused projection in 32-bit:
//   [ q: H*d | k: H*d | v: H*dv | g: H*dv | a: H | b: H ]
#include "common.h"
#include "alice_hip.h"

namespace {

constexpr int THREADS = 256;
constexpr int MAXC = 4;          // value columns a thread owns at most (dv <= MAXC * 256)

__device__ __forceinline__ float logsigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

struct GateNumbers { float keep, put, m_new; };

__device__ __forceinline__ GateNumbers gate_numbers(float a, float b, float cap, float m) {
  const float i = cap > 0.f ? cap * tanhf(a / cap) : a;
  const float f = logsigmoid_f(cap > 0.f ? cap * tanhf(b / cap) : b);
  GateNumbers g;
  g.m_new = fmaxf(f + m, i);
  g.keep = expf(f + m - g.m_new);
  g.put = expf(i - g.m_new);
  return g;
}

// One block per (sequence, head); the sequence's tokens one after the other, the state read from and written
// to memory at every token (element (r, c) of S always by the same thread).  This is the kernel of single
// tokens, and the plain form for any number of them.
template <typename TO>
__global__ __launch_bounds__(THREADS) void mlstm_step_kernel(
    const float* __restrict__ proj, int row_w, const float* __restrict__ bias_i, const float* __restrict__ bias_f,
    const void* __restrict__ norm_w, int norm_dtype, TO* __restrict__ out, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, float* __restrict__ S_all, float* __restrict__ n_all, float* __restrict__ m_all,
    int H, int d, int dv, float cap, float eps, int DG) {
  extern __shared__ float lds[];
  float* qs = lds;                 // d
  float* ks = qs + d;              // d
  float* vs = ks + d;              // dv
  float* part = vs + dv;           // THREADS * MAXC
  __shared__ float red[17];

  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  const int slot = slots[s];
  float* S = S_all + ((size_t)slot * H + h) * d * dv;
  float* nv = n_all + ((size_t)slot * H + h) * d;
  float m = m_all[(size_t)slot * H + h];
  const float qscale = rsqrtf((float)d);
  const int oq = h * d, ok = H * d + h * d, ov = 2 * H * d + h * dv, og = 2 * H * d + H * dv + h * dv;
  const int oa = 2 * H * d + 2 * H * dv + h, ob = oa + H;
  const int G = THREADS / DG, g = tid / DG, j = tid % DG;

  for (int t = t0; t < t1; ++t) {
    const float* row = proj + (size_t)t * row_w;
    __syncthreads();                                   // the last token's reads of qs/ks/vs/part are over
    for (int r = tid; r < d; r += THREADS) { qs[r] = row[oq + r] * qscale; ks[r] = row[ok + r]; }
    for (int c = tid; c < dv; c += THREADS) vs[c] = row[ov + c];
    const GateNumbers gn = gate_numbers(row[oa] + bias_i[h], row[ob] + bias_f[h], cap, m);
    __syncthreads();
    float nq = 0.f;
    for (int r = tid; r < d; r += THREADS) {
      const float x = fmaf(gn.keep, nv[r], gn.put * ks[r]);
      nv[r] = x;
      nq = fmaf(x, qs[r], nq);
    }
    nq = block_sum(nq, red);
    float acc[MAXC];
#pragma unroll
    for (int u = 0; u < MAXC; ++u) {
      acc[u] = 0.f;
      const int c = j + u * DG;
      if (c < dv) {
        const float pv = gn.put * vs[c];
        for (int r = g; r < d; r += G) {
          const float x = fmaf(gn.keep, S[(size_t)r * dv + c], ks[r] * pv);
          S[(size_t)r * dv + c] = x;
          acc[u] = fmaf(x, qs[r], acc[u]);
        }
      }
      part[u * THREADS + tid] = acc[u];
    }
    __syncthreads();
    const float den = fmaxf(fabsf(nq), expf(-gn.m_new)) + 1e-6f;
    float o[MAXC], sq = 0.f;
#pragma unroll
    for (int u = 0; u < MAXC; ++u) {
      o[u] = 0.f;
      const int c = j + u * DG;
      if (g == 0 && c < dv) {
        float x = 0.f;
        for (int gg = 0; gg < G; ++gg) x += part[u * THREADS + gg * DG + j];
        o[u] = x / den;
        sq = fmaf(o[u], o[u], sq);
      }
    }
    sq = block_sum(sq, red);
    const float inv = 1.f / sqrtf(sq / (float)dv + eps);
#pragma unroll
    for (int u = 0; u < MAXC; ++u) {
      const int c = j + u * DG;
      if (g == 0 && c < dv) {
        const float w = norm_dtype == DT_F32 ? ((const float*)norm_w)[h * dv + c] : bf16_to_f32(((const bf16_t*)norm_w)[h * dv + c]);
        const float gate = 1.f / (1.f + expf(-row[og + c]));
        store_f32(out, (size_t)t * H * dv + h * dv + c, o[u] * inv * w * gate);
      }
    }
    m = gn.m_new;
  }
  if (tid == 0 && t1 > t0) m_all[(size_t)slot * H + h] = m;
}

// out[t, j] = gelu_tanh(z[t, j]) * table[tokens[t], col0 + j]: a gate on the rows of a per-token table.
template <typename TZ, typename TW, typename TO, bool FULL>
__global__ void gelu_mul_rows_kernel(const TZ* __restrict__ z, const TW* __restrict__ table, int table_w, int col0,
                                     const int* __restrict__ tokens, TO* __restrict__ out, int n, int V) {
  const int t = blockIdx.x;
  const int tok = tokens[t];
  const bool ok = tok >= 0 && tok < V;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float e = ok ? load_f32(table, (size_t)tok * table_w + col0 + i) : 0.f;
    store_f32(out, (size_t)t * n + i, gelu_tanh_f(load_f32(z, (size_t)t * n + i), FULL) * e);
  }
}

}  // namespace

extern "C" int alice_mlstm_step(const float* proj, int row_w, const float* bias_i, const float* bias_f,
                                const void* norm_w, int norm_dtype, void* out, int out_dtype,
                                const int* cu_seqlens, const int* slots, float* S, float* n, float* m,
                                int n_seqs, int n_slots, int H, int d, int dv, float cap, float eps,
                                hipStream_t stream) {
  ALICE_CHECK(dtype_ok(out_dtype) && dtype_ok(norm_dtype), "mlstm: unknown dtype");
  ALICE_CHECK(n_seqs >= 0 && H >= 1 && H <= 65535 && d >= 1 && dv >= 1, "mlstm: bad sizes H=%d d=%d dv=%d", H, d, dv);
  ALICE_CHECK(dv <= MAXC * THREADS, "mlstm: value head size %d is beyond %d", dv, MAXC * THREADS);
  ALICE_CHECK(row_w >= 2 * H * d + 2 * H * dv + 2 * H, "mlstm: rows of %d numbers are too short", row_w);
  ALICE_CHECK(proj && bias_i && bias_f && norm_w && out && cu_seqlens && slots && S && n && m && n_slots >= 1,
              "mlstm: a pointer is missing");
  if (n_seqs == 0) return 0;
  int DG = 1;
  while (DG < dv && DG < THREADS) DG <<= 1;
  const size_t lds = (size_t)(2 * d + dv + MAXC * THREADS) * sizeof(float);
  ALICE_CHECK(lds <= 64 * 1024, "mlstm: head sizes %d and %d need more shared memory than a block has", d, dv);
  dim3 grid(n_seqs, H);
  if (out_dtype == DT_F32)
    mlstm_step_kernel<float><<<grid, THREADS, lds, stream>>>(proj, row_w, bias_i, bias_f, norm_w, norm_dtype, (float*)out,
        cu_seqlens, slots, S, n, m, H, d, dv, cap, eps, DG);
  else
    mlstm_step_kernel<bf16_t><<<grid, THREADS, lds, stream>>>(proj, row_w, bias_i, bias_f, norm_w, norm_dtype, (bf16_t*)out,
        cu_seqlens, slots, S, n, m, H, d, dv, cap, eps, DG);
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_gelu_mul_rows(const void* z, int z_dtype, const void* table, int table_dtype, int table_w, int col0,
                                   const int* tokens, void* out, int out_dtype, int T, int n, int V,
                                   int full_precision, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(z_dtype) && dtype_ok(table_dtype) && dtype_ok(out_dtype), "gelu_mul_rows: unknown dtype");
  ALICE_CHECK(T >= 0 && n >= 1 && V >= 1 && col0 >= 0 && col0 + n <= table_w, "gelu_mul_rows: columns %d..%d of a table of %d",
              col0, col0 + n, table_w);
  ALICE_CHECK(z_dtype == out_dtype, "gelu_mul_rows: input and output share a dtype");
  if (T == 0) return 0;
  const int threads = n >= 256 ? 256 : (n >= 128 ? 128 : 64);
#define GO(TZ, TW, FULL) gelu_mul_rows_kernel<TZ, TW, TZ, FULL><<<T, threads, 0, stream>>>((const TZ*)z, (const TW*)table, table_w, col0, tokens, (TZ*)out, n, V)
  if (z_dtype == DT_F32) {
    if (table_dtype == DT_F32) { if (full_precision) GO(float, float, true); else GO(float, float, false); }
    else { if (full_precision) GO(float, bf16_t, true); else GO(float, bf16_t, false); }
  } else {
    if (table_dtype == DT_F32) { if (full_precision) GO(bf16_t, float, true); else GO(bf16_t, float, false); }
    else { if (full_precision) GO(bf16_t, bf16_t, true); else GO(bf16_t, bf16_t, false); }
  }
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}
