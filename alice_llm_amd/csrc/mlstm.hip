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

typedef float f32x4_t __attribute__((ext_vector_type(4)));
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


// ------------------------------------------------------------------------------------------------ chunks
// The same recurrence for many tokens of a sequence, a chunk of C tokens at a time.  Inside a chunk, with
// b_j the running sum of the log forget gates, a_r = i_r - b_r and M_j = max(m_0, max_{r <= j} a_r) (m_0: the
// stabiliser before the chunk), the token-by-token definition gives m_j = b_j + M_j and
//   S_j = exp(m_0 - M_j) S_0 + sum_{r <= j} exp(a_r - M_j) k_r v_r^T          (n_j alike),
// so that  S_j^T q_j = exp(m_0 - M_j) (Q S_0)_j + ((Q K^T . D) V)_j  with  D_jr = exp(a_r - M_j), r <= j.
// Four matrix products a chunk (Q K^T, Q S_0, P V, K'^T V), all on the 32-bit matrix instruction
// (v_mfma_f32_16x16x4_f32): the state, the gates' weights and everything they multiply stay 32-bit.
// A block owns VS of a head's value columns (S's columns are independent of each other) for all chunks of
// one sequence; blocks of one head recompute its gates and Q K^T.  The head norm needs every column, so the
// read-outs go to a 32-bit workspace and mlstm_finish_kernel norms, weights and gates them.

// Row strides in LDS, for 32 banks of four bytes read by half a wave at a time.  Q, K and P rows are read as
// 16 rows x 2 neighbours (operand A, and K as operand B of Q K^T), and K also as 2 rows x 16 neighbours (K'^T V):
// a stride of 18 mod 32 serves the first without conflicts and the second with two banks shared.  V and S rows
// are read as 2 rows x 16 neighbours only: 16 mod 32.
__host__ __device__ __forceinline__ int lds_stride18(int d) { return d + ((18 - d % 32 + 32) % 32); }

// A barrier between phases that exchange data through LDS only: it waits for the wave's LDS accesses, not for its
// loads and stores of global memory (the rows fetched ahead, the read-outs on their way out), which __syncthreads()
// would also wait for at every phase.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// acc += sum over k < n (a multiple of 16) of A(k) B(k), four k at a time, as four chains of products that do not
// wait for each other (a product that adds to the one before it waits for its result, about twice the time the
// matrix unit is busy with it); the chains are added at the end.
template <class FA, class FB>
__device__ __forceinline__ void mfma_chains(f32x4_t& acc, int n, FA a, FB b) {
  f32x4_t c1 = {0.f, 0.f, 0.f, 0.f}, c2 = c1, c3 = c1;
#pragma unroll 2
  for (int kk = 0; kk < n; kk += 16) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a(kk), b(kk), acc, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a(kk + 4), b(kk + 4), c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a(kk + 8), b(kk + 8), c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_16x16x4f32(a(kk + 12), b(kk + 12), c3, 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] += (c1[i] + c2[i]) + c3[i];
}

constexpr int CTHREADS = 512;     // eight waves a block: two a SIMD, so that one's LDS reads hide behind the other's products
constexpr int CWAVES = CTHREADS / 64;

// MODE 0: a block walks all chunks of its sequence, from and to the cache's state (grid.x: sequences).
// For steps whose sequences x heads x slices leave the chip unfilled, the chunks run side by side instead
// (grid.x: sequences x max_chunks): MODE 1 leaves every chunk's own sums, from an empty state, in the workspace
// (U = K'^T V with weights exp(a_r - A), A = max_r a_r; u_n alike; A and the chunk's sum of log forget gates);
// mlstm_chunk_states_kernel walks the chunks' sums and leaves the state and stabiliser before every chunk in
// their place; MODE 2 takes every chunk's read-outs from the state before it.
struct ChunkSpace { float* S; float* n; float* sc; float* m0; int max_chunks; };

template <int C, int VS, int MODE>
__global__ __launch_bounds__(CTHREADS) void mlstm_chunk_kernel(
    const float* __restrict__ proj, int row_w, const float* __restrict__ bias_i, const float* __restrict__ bias_f,
    float* __restrict__ work, float* __restrict__ dens, const int* __restrict__ cu_seqlens, const int* __restrict__ slots,
    float* __restrict__ S_all, float* __restrict__ n_all, float* __restrict__ m_all,
    int H, int d, int dv, float cap, ChunkSpace ws) {
  constexpr int VSS = VS == 16 ? 16 : VS + 16; // row stride of V and S tiles: 16 mod 32 banks
  constexpr int PSS = C + 2;
  constexpr int CT = C / 16, VT = VS / 16;
  extern __shared__ float lds[];
  const int QS = lds_stride18(d);
  float* Qs = lds;                       // [C][QS]
  float* Ks = Qs + C * QS;               // [C][QS]
  float* Vs = Ks + C * QS;               // [C][VSS]
  float* Ps = Vs + C * VSS;              // [C][PSS]
  float* Ss = Ps + C * PSS;              // [d][VSS]
  float* n0 = Ss + d * VSS;              // [d]
  float* ga = n0 + d;                    // [C] a_r
  float* gM = ga + C;                    // [C] M_j
  float* gm = gM + C;                    // [C] m_j
  float* gcoef = gm + C;                 // [C] exp(m_0 - M_j)
  float* gw = gcoef + C;                 // [C] exp(a_r - M_last)

  const int s = MODE == 0 ? blockIdx.x : blockIdx.x / ws.max_chunks, chunk = MODE == 0 ? 0 : blockIdx.x % ws.max_chunks;
  const int h = blockIdx.y, v0 = blockIdx.z * VS, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  const int c_begin = t0 + chunk * C, c_end = MODE == 0 ? t1 : min(t1, c_begin + C);
  if (c_end <= c_begin) return;
  const int slot = slots[s];
  const size_t cid = (size_t)blockIdx.x * H + h;             // the chunk's place in the workspace (MODE 1, 2)
  float* Sg = MODE == 0 ? S_all + ((size_t)slot * H + h) * d * dv : ws.S + cid * d * dv;
  float* ng = MODE == 0 ? n_all + ((size_t)slot * H + h) * d : ws.n + cid * d;
  float m0 = MODE == 0 ? m_all[(size_t)slot * H + h] : (MODE == 1 ? -INFINITY : ws.m0[cid]);
  float M_end = 0.f;
  const float qscale = rsqrtf((float)d);
  const int oq = h * d, ok = H * d + h * d, ov = 2 * H * d + h * dv + v0;
  const int oa = 2 * H * d + 2 * H * dv + h, ob = oa + H;
  const float bi = bias_i[h], bf = bias_f[h];

  for (int i = tid; i < d * VS; i += CTHREADS) Ss[(i / VS) * VSS + i % VS] = MODE == 1 ? 0.f : Sg[(size_t)(i / VS) * dv + v0 + i % VS];
  for (int r = tid; r < d; r += CTHREADS) n0[r] = MODE == 1 ? 0.f : ng[r];

  // A chunk's rows are fetched into registers while the chunk before is worked on, and its gates' tanh and
  // logarithm are taken by wave 0 at the end of that chunk: neither waits in a chunk's own time.
  constexpr int NQ = 4, NV = 2;                          // float4s a thread fetches at most (checked by the host's plan)
  const int q4 = C * (d / 4);
  float4 rq[NQ], rk[NQ], rv[NV];
  float raw_a = 0.f, raw_b = 0.f, ig_n = -INFINITY, fg_n = 0.f;
  auto fetch = [&](int c0) {
    const int len = min(C, t1 - c0);
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int i = tid + u * CTHREADS;
      const int j = i / (d / 4), k = (i % (d / 4)) * 4;
      rq[u] = rk[u] = float4{0.f, 0.f, 0.f, 0.f};
      if (i < q4 && j < len) {
        const float* row = proj + (size_t)(c0 + j) * row_w;
        rq[u] = *reinterpret_cast<const float4*>(row + oq + k);
        rk[u] = *reinterpret_cast<const float4*>(row + ok + k);
      }
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int i = tid + u * CTHREADS;
      const int j = i / (VS / 4), k = (i % (VS / 4)) * 4;
      rv[u] = float4{0.f, 0.f, 0.f, 0.f};
      if (i < C * (VS / 4) && j < len) rv[u] = *reinterpret_cast<const float4*>(proj + (size_t)(c0 + j) * row_w + ov + k);
    }
    if (wave == 0 && lane < len) {
      const float* row = proj + (size_t)(c0 + lane) * row_w;
      raw_a = row[oa];
      raw_b = row[ob];
    }
  };
  auto gates_ahead = [&](int c0) {                       // wave 0: the log gates of the fetched chunk
    ig_n = -INFINITY;
    fg_n = 0.f;
    if (lane < min(C, t1 - c0)) {
      const float a = raw_a + bi, b = raw_b + bf;
      ig_n = cap > 0.f ? cap * tanhf(a / cap) : a;
      fg_n = logsigmoid_f(cap > 0.f ? cap * tanhf(b / cap) : b);
    }
  };
  fetch(c_begin);
  if (wave == 0) gates_ahead(c_begin);

  for (int c0 = c_begin; c0 < c_end; c0 += C) {
    const int len = min(C, t1 - c0);
    lds_barrier();                                     // the chunk before is done with every buffer
    // ---- phase 1: the fetched rows into LDS, the gates' running sums and maxima
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int i = tid + u * CTHREADS;
      if (i < q4) {
        const int j = i / (d / 4), k = (i % (d / 4)) * 4;
        float2* qd = reinterpret_cast<float2*>(Qs + j * QS + k);      // rows start at multiples of 8 bytes
        float2* kd = reinterpret_cast<float2*>(Ks + j * QS + k);
        qd[0] = float2{rq[u].x * qscale, rq[u].y * qscale};
        qd[1] = float2{rq[u].z * qscale, rq[u].w * qscale};
        kd[0] = float2{rk[u].x, rk[u].y};
        kd[1] = float2{rk[u].z, rk[u].w};
      }
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int i = tid + u * CTHREADS;
      if (i < C * (VS / 4)) *reinterpret_cast<float4*>(Vs + (i / (VS / 4)) * VSS + (i % (VS / 4)) * 4) = rv[u];
    }
    if (wave == 0) {
      float b = fg_n;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) { const float t = __shfl_up(b, o, 64); if (lane >= o) b += t; }
      const float a = ig_n - b;
      float M = a;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) { const float t = __shfl_up(M, o, 64); if (lane >= o) M = fmaxf(M, t); }
      M = fmaxf(M, m0);
      if (lane < C) { ga[lane] = a; gM[lane] = M; gm[lane] = b + M; gcoef[lane] = expf(m0 - M); }
    }
    const bool more = c0 + C < c_end;
    if (more) fetch(c0 + C);
    lds_barrier();
    const float M_last = gM[len - 1], m_last = gm[len - 1];
    // ---- phase 2: P = (Q K^T) . D on and below the diagonal
    for (int tile = wave; tile < (MODE == 1 ? 0 : CT * (CT + 1) / 2); tile += CWAVES) {
      int ti = 0, rem = tile;
      while (rem > ti) { rem -= ti + 1; ++ti; }
      const int tj = rem;
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
      const float* qa = Qs + (ti * 16 + (lane & 15)) * QS + (lane >> 4);
      const float* kb = Ks + (tj * 16 + (lane & 15)) * QS + (lane >> 4);
      mfma_chains(acc, d, [&](int k) { return qa[k]; }, [&](int k) { return kb[k]; });
      const int r = tj * 16 + (lane & 15);
      const float ar = ga[r];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = ti * 16 + (lane >> 4) * 4 + i;
        const float w = r <= j ? expf(ar - gM[j]) : 0.f;
        Ps[j * PSS + r] = acc[i] * w;
      }
    }
    if (tid < C) gw[tid] = tid < len ? expf(ga[tid] - M_last) : 0.f;
    lds_barrier();
    // ---- phase 3: read-outs coef . Q S_0 + P V, unnormalised; the blocks of a head's first columns also take
    // n . q the same way (n as one more column: Q n_0 and the row sums of P) and leave the denominators
    const int n_tiles3 = MODE == 1 ? 0 : CT * VT + (blockIdx.z == 0 ? CT : 0);
    for (int tile = wave; tile < n_tiles3; tile += CWAVES) {
      const bool is_n = tile >= CT * VT;
      const int ti = is_n ? tile - CT * VT : tile / VT, tn = is_n ? 0 : tile % VT;
      const bool col0 = (lane & 15) == 0;
      f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
      const float* qa = Qs + (ti * 16 + (lane & 15)) * QS + (lane >> 4);
      const float* pa = Ps + (ti * 16 + (lane & 15)) * PSS + (lane >> 4);
      if (!is_n) {
        const float* sb = Ss + (lane >> 4) * VSS + tn * 16 + (lane & 15);
        mfma_chains(acc, d, [&](int k) { return qa[k]; }, [&](int k) { return sb[k * VSS]; });
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] *= gcoef[ti * 16 + (lane >> 4) * 4 + i];
        const float* vb = Vs + (lane >> 4) * VSS + tn * 16 + (lane & 15);
        mfma_chains(acc, (ti + 1) * 16, [&](int k) { return pa[k]; }, [&](int k) { return vb[k * VSS]; });
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = ti * 16 + (lane >> 4) * 4 + i;
          if (j < len) work[(size_t)(c0 + j) * H * dv + h * dv + v0 + tn * 16 + (lane & 15)] = acc[i];
        }
      } else {
        const float* nb = n0 + (lane >> 4);
        mfma_chains(acc, d, [&](int k) { return qa[k]; }, [&](int k) { return col0 ? nb[k] : 0.f; });
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] *= gcoef[ti * 16 + (lane >> 4) * 4 + i];
        const float one = col0 ? 1.f : 0.f;
        mfma_chains(acc, (ti + 1) * 16, [&](int k) { return pa[k]; }, [&](int) { return one; });
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = ti * 16 + (lane >> 4) * 4 + i;
          if (col0 && j < len) dens[(size_t)(c0 + j) * H + h] = fmaxf(fabsf(acc[i]), expf(-gm[j])) + 1e-6f;
        }
      }
    }
    lds_barrier();                                     // every read of S_0 and n_0 is over
    // ---- phase 4: the state at the chunk's end (n again as one more column)
    const float cS = expf(m0 - M_last);
    const int n_tiles4 = MODE == 2 ? 0 : (d / 16) * VT + (blockIdx.z == 0 ? d / 16 : 0);
    for (int tile = wave; tile < n_tiles4; tile += CWAVES) {
      const bool is_n = tile >= (d / 16) * VT;
      const int tk = is_n ? tile - (d / 16) * VT : tile / VT, tn = is_n ? 0 : tile % VT;
      const bool col0 = (lane & 15) == 0;
      const float* ka = Ks + (lane >> 4) * QS + tk * 16 + (lane & 15);
      f32x4_t acc;
      if (!is_n) {
        float* sp = Ss + (tk * 16 + (lane >> 4) * 4) * VSS + tn * 16 + (lane & 15);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = cS * sp[i * VSS];
        const float* vb = Vs + (lane >> 4) * VSS + tn * 16 + (lane & 15);
        mfma_chains(acc, C, [&](int k) { return ka[k * QS] * gw[k + (lane >> 4)]; }, [&](int k) { return vb[k * VSS]; });
#pragma unroll
        for (int i = 0; i < 4; ++i) sp[i * VSS] = acc[i];
      } else {
        float* np = n0 + tk * 16 + (lane >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = col0 ? cS * np[i] : 0.f;
        const float one = col0 ? 1.f : 0.f;
        mfma_chains(acc, C, [&](int k) { return ka[k * QS] * gw[k + (lane >> 4)]; }, [&](int) { return one; });
        if (col0) {
#pragma unroll
          for (int i = 0; i < 4; ++i) np[i] = acc[i];
        }
      }
    }
    m0 = m_last;
    M_end = M_last;
    if (more && wave == 0) gates_ahead(c0 + C);
  }
  if (MODE == 2) return;
  __syncthreads();
  for (int i = tid; i < d * VS; i += CTHREADS) Sg[(size_t)(i / VS) * dv + v0 + i % VS] = Ss[(i / VS) * VSS + i % VS];
  if (blockIdx.z == 0) {
    for (int r = tid; r < d; r += CTHREADS) ng[r] = n0[r];
    if (tid == 0) {
      if (MODE == 0) m_all[(size_t)slot * H + h] = m0;
      else { ws.sc[cid * 2] = M_end; ws.sc[cid * 2 + 1] = m0 - M_end; }      // A, and the sum of the log forget gates
    }
  }
}

// Between MODE 1 and MODE 2: per (sequence, head) the chunks one after the other, element by element.  With the
// state s and stabiliser m before chunk c, and the chunk's own sums u, A and b: the state before the chunk goes
// where u was; then M = max(m, A), s <- exp(m - M) s + exp(A - M) u, m <- b + M.  The end state goes to the cache.
__global__ __launch_bounds__(THREADS) void mlstm_chunk_states_kernel(
    const int* __restrict__ cu_seqlens, const int* __restrict__ slots, float* __restrict__ S_all,
    float* __restrict__ n_all, float* __restrict__ m_all, int H, int d, int dv, int C, ChunkSpace ws) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  if (t1 <= t0) return;
  const int n_chunks = (t1 - t0 + C - 1) / C;
  const int slot = slots[s];
  const size_t per = (size_t)d * dv;
  const size_t e = ((size_t)blockIdx.z * THREADS + threadIdx.x) * 4;       // four elements a thread
  const bool does_n = blockIdx.z == 0 && threadIdx.x < (d + 3) / 4;        // and the first block the vector n too
  float4 st = {0.f, 0.f, 0.f, 0.f}, nn = st;
  float* Sg = S_all + ((size_t)slot * H + h) * per;
  float* ng = n_all + ((size_t)slot * H + h) * d;
  if (e < per) st = *reinterpret_cast<const float4*>(Sg + e);
  if (does_n) nn = *reinterpret_cast<const float4*>(ng + threadIdx.x * 4);
  float m = m_all[(size_t)slot * H + h];
  for (int c0 = 0; c0 < n_chunks; c0 += 4) {
    float4 u[4], un[4];
    float A[4], b[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {                               // the loads of four chunks before the first use
      const size_t cid = ((size_t)s * ws.max_chunks + min(c0 + k, n_chunks - 1)) * H + h;
      u[k] = e < per ? *reinterpret_cast<const float4*>(ws.S + cid * per + e) : float4{0.f, 0.f, 0.f, 0.f};
      un[k] = does_n ? *reinterpret_cast<const float4*>(ws.n + cid * d + threadIdx.x * 4) : float4{0.f, 0.f, 0.f, 0.f};
      A[k] = ws.sc[cid * 2];
      b[k] = ws.sc[cid * 2 + 1];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (c0 + k < n_chunks) {
        const size_t cid = ((size_t)s * ws.max_chunks + c0 + k) * H + h;
        if (e < per) *reinterpret_cast<float4*>(ws.S + cid * per + e) = st;
        if (does_n) *reinterpret_cast<float4*>(ws.n + cid * d + threadIdx.x * 4) = nn;
        if (blockIdx.z == 0 && threadIdx.x == 0) ws.m0[cid] = m;
        const float M = fmaxf(m, A[k]);
        const float ka = expf(m - M), kb = expf(A[k] - M);
        st = float4{ka * st.x + kb * u[k].x, ka * st.y + kb * u[k].y, ka * st.z + kb * u[k].z, ka * st.w + kb * u[k].w};
        nn = float4{ka * nn.x + kb * un[k].x, ka * nn.y + kb * un[k].y, ka * nn.z + kb * un[k].z, ka * nn.w + kb * un[k].w};
        m = b[k] + M;
      }
    }
  }
  if (e < per) *reinterpret_cast<float4*>(Sg + e) = st;
  if (does_n) *reinterpret_cast<float4*>(ng + threadIdx.x * 4) = nn;
  if (blockIdx.z == 0 && threadIdx.x == 0) m_all[(size_t)slot * H + h] = m;
}


// Single tokens (and pieces of a few): a block per (sequence, head, 64 value columns).  Lane l of every wave owns
// column c = 64 z + l; wave w owns the rows r = w, w + 4, ...; a thread keeps its RPT elements of S in registers
// over the sequence's tokens, so the state is read once and written once, in 256-byte runs.  The head norm needs
// every column: the read-outs go to the 32-bit workspace and mlstm_finish_kernel does the rest.
template <int RPT>
__global__ __launch_bounds__(THREADS) void mlstm_cols_kernel(
    const float* __restrict__ proj, int row_w, const float* __restrict__ bias_i, const float* __restrict__ bias_f,
    float* __restrict__ work, const int* __restrict__ cu_seqlens, const int* __restrict__ slots,
    float* __restrict__ S_all, float* __restrict__ n_all, float* __restrict__ m_all,
    int H, int d, int dv, float cap) {
  extern __shared__ float lds[];
  float* qs = lds;                 // d
  float* ks = qs + d;              // d
  float* ns = ks + d;              // d
  float* part = ns + d;            // 4 * 64
  __shared__ float red[17];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int c = blockIdx.z * 64 + lane;
  const bool col = c < dv;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  if (t1 <= t0) return;
  const int slot = slots[s];
  float* S = S_all + ((size_t)slot * H + h) * d * dv;
  float* ng = n_all + ((size_t)slot * H + h) * d;
  float m = m_all[(size_t)slot * H + h];
  float st[RPT];
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = w + 4 * i;
    st[i] = (col && r < d) ? S[(size_t)r * dv + c] : 0.f;
  }
  for (int r = tid; r < d; r += THREADS) ns[r] = ng[r];
  const float qscale = rsqrtf((float)d);
  const int oq = h * d, ok = H * d + h * d, ov = 2 * H * d + h * dv;
  const int oa = 2 * H * d + 2 * H * dv + h, ob = oa + H;
  const float bi = bias_i[h], bf = bias_f[h];
  for (int t = t0; t < t1; ++t) {
    const float* row = proj + (size_t)t * row_w;
    __syncthreads();
    for (int r = tid; r < d; r += THREADS) { qs[r] = row[oq + r] * qscale; ks[r] = row[ok + r]; }
    const float v = col ? row[ov + c] : 0.f;
    const GateNumbers gn = gate_numbers(row[oa] + bi, row[ob] + bf, cap, m);
    __syncthreads();
    float nq = 0.f;
    for (int r = tid; r < d; r += THREADS) {
      const float x = fmaf(gn.keep, ns[r], gn.put * ks[r]);
      ns[r] = x;
      nq = fmaf(x, qs[r], nq);
    }
    nq = block_sum(nq, red);
    const float pv = gn.put * v;
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int r = w + 4 * i;
      if (r < d) {
        st[i] = fmaf(gn.keep, st[i], ks[r] * pv);
        acc = fmaf(st[i], qs[r], acc);
      }
    }
    part[w * 64 + lane] = acc;
    __syncthreads();
    if (w == 0 && col) {
      const float den = fmaxf(fabsf(nq), expf(-gn.m_new)) + 1e-6f;
      work[(size_t)t * H * dv + h * dv + c] = (part[lane] + part[64 + lane] + part[128 + lane] + part[192 + lane]) / den;
    }
    m = gn.m_new;
  }
#pragma unroll
  for (int i = 0; i < RPT; ++i) {
    const int r = w + 4 * i;
    if (col && r < d) S[(size_t)r * dv + c] = st[i];
  }
  if (blockIdx.z == 0) {
    __syncthreads();
    for (int r = tid; r < d; r += THREADS) ng[r] = ns[r];
    if (tid == 0) m_all[(size_t)slot * H + h] = m;
  }
}


// Single tokens with value heads of up to 256 and keys of up to 128: a block per (sequence, head), a thread per
// value column with the column's d elements of S in registers.  The head's read-out is whole inside the block, so
// the head norm, its weight and the output gate follow at once: one kernel a step, the state read and written once.
template <int DMAX, typename TO>
__global__ __launch_bounds__(THREADS) void mlstm_head_kernel(
    const float* __restrict__ proj, int row_w, const float* __restrict__ bias_i, const float* __restrict__ bias_f,
    const void* __restrict__ norm_w, int norm_dtype, TO* __restrict__ out, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, float* __restrict__ S_all, float* __restrict__ n_all, float* __restrict__ m_all,
    int H, int d, int dv, float cap, float eps) {
  extern __shared__ float lds[];
  float* qs = lds;                 // d
  float* ks = qs + d;              // d
  float* ns = ks + d;              // d
  __shared__ float red[17];
  const int s = blockIdx.x, h = blockIdx.y, c = threadIdx.x;
  const bool col = c < dv;
  const int t0 = cu_seqlens[s], t1 = cu_seqlens[s + 1];
  if (t1 <= t0) return;
  const int slot = slots[s];
  float* S = S_all + ((size_t)slot * H + h) * d * dv;
  float* ng = n_all + ((size_t)slot * H + h) * d;
  float m = m_all[(size_t)slot * H + h];
  float st[DMAX];
#pragma unroll
  for (int r = 0; r < DMAX; ++r) st[r] = (col && r < d) ? S[(size_t)r * dv + c] : 0.f;
  for (int r = c; r < d; r += blockDim.x) ns[r] = ng[r];
  const float qscale = rsqrtf((float)d);
  const int oq = h * d, ok = H * d + h * d, ov = 2 * H * d + h * dv, og = 2 * H * d + H * dv + h * dv;
  const int oa = 2 * H * d + 2 * H * dv + h, ob = oa + H;
  const float bi = bias_i[h], bf = bias_f[h];
  const float w = !col ? 0.f : norm_dtype == DT_F32 ? ((const float*)norm_w)[h * dv + c] : bf16_to_f32(((const bf16_t*)norm_w)[h * dv + c]);
  for (int t = t0; t < t1; ++t) {
    const float* row = proj + (size_t)t * row_w;
    __syncthreads();
    for (int r = c; r < d; r += blockDim.x) { qs[r] = row[oq + r] * qscale; ks[r] = row[ok + r]; }
    const float v = col ? row[ov + c] : 0.f, g = col ? row[og + c] : 0.f;
    const GateNumbers gn = gate_numbers(row[oa] + bi, row[ob] + bf, cap, m);
    __syncthreads();
    float nq = 0.f;
    for (int r = c; r < d; r += blockDim.x) {
      const float x = fmaf(gn.keep, ns[r], gn.put * ks[r]);
      ns[r] = x;
      nq = fmaf(x, qs[r], nq);
    }
    nq = block_sum(nq, red);
    const float pv = gn.put * v;
    float acc = 0.f;
#pragma unroll
    for (int r = 0; r < DMAX; ++r) {
      if (r < d) {
        st[r] = fmaf(gn.keep, st[r], ks[r] * pv);
        acc = fmaf(st[r], qs[r], acc);
      }
    }
    const float o = col ? acc / (fmaxf(fabsf(nq), expf(-gn.m_new)) + 1e-6f) : 0.f;
    const float sq = block_sum(o * o, red);
    if (col) store_f32(out, (size_t)t * H * dv + h * dv + c, o / sqrtf(sq / (float)dv + eps) * w / (1.f + expf(-g)));
    m = gn.m_new;
  }
#pragma unroll
  for (int r = 0; r < DMAX; ++r)
    if (col && r < d) S[(size_t)r * dv + c] = st[r];
  __syncthreads();
  for (int r = c; r < d; r += blockDim.x) ng[r] = ns[r];
  if (c == 0) m_all[(size_t)slot * H + h] = m;
}

// With o = work[t, h, :] (divided by dens[t, h] where the read-outs were left unnormalised):
// out[t, h, :] = o / rms(o) * w[h, :] * sigmoid(g[t, h, :]); a block per (token, head).
template <typename TO>
__global__ void mlstm_finish_kernel(const float* __restrict__ work, const float* __restrict__ dens,
                                    const float* __restrict__ proj, int row_w,
                                    const void* __restrict__ norm_w, int norm_dtype, TO* __restrict__ out,
                                    int H, int d, int dv, float eps) {
  __shared__ float red[17];
  const int t = blockIdx.x, h = blockIdx.y;
  const float* o = work + (size_t)t * H * dv + h * dv;
  const float* g = proj + (size_t)t * row_w + 2 * H * d + H * dv + h * dv;
  const float den = dens ? dens[(size_t)t * H + h] : 1.f;
  float sq = 0.f;
  for (int c = threadIdx.x; c < dv; c += blockDim.x) { const float x = o[c] / den; sq = fmaf(x, x, sq); }
  sq = block_sum(sq, red);
  const float inv = 1.f / sqrtf(sq / (float)dv + eps);
  for (int c = threadIdx.x; c < dv; c += blockDim.x) {
    const float w = norm_dtype == DT_F32 ? ((const float*)norm_w)[h * dv + c] : bf16_to_f32(((const bf16_t*)norm_w)[h * dv + c]);
    store_f32(out, (size_t)t * H * dv + h * dv + c, o[c] / den * inv * w / (1.f + expf(-g[c])));
  }
}

size_t chunk_lds_bytes(int C, int VS, int d) {
  const int QS = lds_stride18(d), VSS = VS == 16 ? 16 : VS + 16;
  return (size_t)(2 * C * QS + C * VSS + C * (C + 2) + d * VSS + d + 5 * C) * sizeof(float);
}

// The chunk length and the columns a block owns for these sizes (0, 0: the chunk kernel does not cover them).
void chunk_plan(int n_seqs, int H, int d, int dv, int* C, int* VS) {
  *C = *VS = 0;
  if (d % 16 || dv % 16 || d > 256) return;
  const int c = d <= 128 ? 64 : 32;
  int best = 0;
  for (int vs = 64; vs >= 16; vs >>= 1) {
    if (dv % vs || (c == 32 && vs == 64) || chunk_lds_bytes(c, vs, d) > 150 * 1024) continue;
    if (c * (d / 4) > 4 * CTHREADS || c * (vs / 4) > 2 * CTHREADS) continue;        // what a thread fetches ahead
    if (!best) best = vs;
    if ((long)n_seqs * H * (dv / best) >= 256) break;      // the widest slice that still makes a block a CU
    best = vs;
  }
  if (best) { *C = c; *VS = best; }
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

// alice_mlstm_step's result for key sizes up to 256 with the state read and written once a step: a block a head
// where the head fits one (keys up to 128, values up to 256), else blocks of 64 value columns and a finishing
// kernel; work: float32 [T, H * dv].
extern "C" int alice_mlstm_cols(const float* proj, int row_w, const float* bias_i, const float* bias_f,
                                const void* norm_w, int norm_dtype, void* out, int out_dtype, float* work,
                                const int* cu_seqlens, const int* slots, float* S, float* n, float* m,
                                int T, int n_seqs, int n_slots, int H, int d, int dv, float cap, float eps,
                                hipStream_t stream) {
  ALICE_CHECK(dtype_ok(out_dtype) && dtype_ok(norm_dtype), "mlstm: unknown dtype");
  ALICE_CHECK(T >= 0 && n_seqs >= 0 && H >= 1 && H <= 65535 && d >= 1 && d <= 256 && dv >= 1 && dv <= 64 * 65535,
              "mlstm: bad sizes H=%d d=%d dv=%d (keys up to 256 here)", H, d, dv);
  ALICE_CHECK(row_w >= 2 * H * d + 2 * H * dv + 2 * H, "mlstm: rows of %d numbers are too short", row_w);
  ALICE_CHECK(proj && bias_i && bias_f && norm_w && out && work && cu_seqlens && slots && S && n && m && n_slots >= 1,
              "mlstm: a pointer is missing");
  if (n_seqs == 0 || T == 0) return 0;
  // The whole head in one block (no workspace, no second kernel) where such blocks fill the chip; with fewer, a
  // CU's own share of the memory rate bounds a block that moves a whole head's state (batch 8 of 8 heads: 24 us
  // against 11 + 9 for the two kernels below).
  if (d <= 128 && dv <= THREADS && (long)n_seqs * H >= 256) {
    const int threads = (dv + 63) / 64 * 64;
    const size_t lds1 = (size_t)3 * d * sizeof(float);
#define GO1(D, TT) mlstm_head_kernel<D, TT><<<dim3(n_seqs, H), threads, lds1, stream>>>(proj, row_w, bias_i, bias_f, norm_w, norm_dtype, (TT*)out, cu_seqlens, slots, S, n, m, H, d, dv, cap, eps)
    if (out_dtype == DT_F32) { if (d <= 32) GO1(32, float); else if (d <= 64) GO1(64, float); else GO1(128, float); }
    else { if (d <= 32) GO1(32, bf16_t); else if (d <= 64) GO1(64, bf16_t); else GO1(128, bf16_t); }
#undef GO1
    ALICE_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid(n_seqs, H, (dv + 63) / 64);
  const size_t lds = (size_t)(3 * d + 256) * sizeof(float);
#define GO(R) mlstm_cols_kernel<R><<<grid, THREADS, lds, stream>>>(proj, row_w, bias_i, bias_f, work, cu_seqlens, slots, S, n, m, H, d, dv, cap)
  if (d <= 64) GO(16);
  else if (d <= 128) GO(32);
  else GO(64);
#undef GO
  ALICE_LAUNCH_CHECK();
  const int threads = dv >= 256 ? 256 : (dv >= 128 ? 128 : 64);
  if (out_dtype == DT_F32)
    mlstm_finish_kernel<float><<<dim3(T, H), threads, 0, stream>>>(work, nullptr, proj, row_w, norm_w, norm_dtype, (float*)out, H, d, dv, eps);
  else
    mlstm_finish_kernel<bf16_t><<<dim3(T, H), threads, 0, stream>>>(work, nullptr, proj, row_w, norm_w, norm_dtype, (bf16_t*)out, H, d, dv, eps);
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_mlstm_chunks_supported(int n_seqs, int H, int d, int dv) {
  int C, VS;
  chunk_plan(n_seqs, H, d, dv, &C, &VS);
  return C != 0;
}

// The same as alice_mlstm_step for steps of many tokens a sequence, a chunk at a time on the matrix cores;
// work: alice_mlstm_chunks_workspace(...) float32; max_new: the most tokens of one sequence in the step.  Sizes it
// does not cover (alice_mlstm_chunks_supported) are refused.
extern "C" long alice_mlstm_chunks_workspace(int T, int n_seqs, int max_new, int H, int d, int dv) {
  int C, VS;
  chunk_plan(n_seqs, H, d, dv, &C, &VS);
  long n = (long)T * ((long)H * dv + H);
  if (C && max_new > C && (long)n_seqs * H * (dv / 16) < 256)           // the chunks side by side: their states too
    n += 4 + (long)n_seqs * ((max_new + C - 1) / C) * H * ((long)d * dv + d + 3);
  return n;
}

extern "C" int alice_mlstm_chunks(const float* proj, int row_w, const float* bias_i, const float* bias_f,
                                  const void* norm_w, int norm_dtype, void* out, int out_dtype, float* work,
                                  const int* cu_seqlens, const int* slots, float* S, float* n, float* m,
                                  int T, int n_seqs, int n_slots, int H, int d, int dv, float cap, float eps,
                                  int max_new, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(out_dtype) && dtype_ok(norm_dtype), "mlstm: unknown dtype");
  ALICE_CHECK(T >= 0 && n_seqs >= 0 && H >= 1 && H <= 65535 && d >= 1 && dv >= 1, "mlstm: bad sizes H=%d d=%d dv=%d", H, d, dv);
  ALICE_CHECK(row_w >= 2 * H * d + 2 * H * dv + 2 * H && row_w % 4 == 0 && ((uintptr_t)proj & 15) == 0,
              "mlstm: rows of %d numbers are too short, or not a multiple of four numbers from a 16-byte boundary", row_w);
  ALICE_CHECK(proj && bias_i && bias_f && norm_w && out && work && cu_seqlens && slots && S && n && m && n_slots >= 1,
              "mlstm: a pointer is missing");
  ALICE_CHECK(max_new >= 1 && max_new <= T, "mlstm: the longest piece of the step, %d tokens, is outside 1..%d", max_new, T);
  int C, VS;
  chunk_plan(n_seqs, H, d, dv, &C, &VS);
  ALICE_CHECK(C != 0, "mlstm: the chunk kernel does not cover head sizes %d and %d", d, dv);
  if (n_seqs == 0 || T == 0) return 0;
  float* dens = work + (size_t)T * H * dv;               // the denominators, [T, H], behind the read-outs
  const bool side_by_side = max_new > C && (long)n_seqs * H * (dv / 16) < 256;
  ChunkSpace ws = {nullptr, nullptr, nullptr, nullptr, 1};
  if (side_by_side) {
    ws.max_chunks = (max_new + C - 1) / C;
    const size_t nc = (size_t)n_seqs * ws.max_chunks * H;
    ws.S = dens + (((size_t)T * H + 3) & ~(size_t)3);          // 16-byte aligned
    ws.n = ws.S + nc * d * dv;
    ws.sc = ws.n + nc * d;
    ws.m0 = ws.sc + nc * 2;
    chunk_plan(n_seqs * ws.max_chunks, H, d, dv, &C, &VS);          // the slices for that many blocks (C is the same)
  }
  const size_t lds = chunk_lds_bytes(C, VS, d);
#define GO_MODE(CC, VV, MODE, GX)                                                                                    \
  do {                                                                                                               \
    static bool raised = false; /* blocks of more than 64 KB of shared memory: said once per kernel */              \
    if (!raised) {                                                                                                   \
      hipFuncSetAttribute((const void*)mlstm_chunk_kernel<CC, VV, MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
      (void)hipGetLastError();                                                                                       \
      raised = true;                                                                                                 \
    }                                                                                                                \
    mlstm_chunk_kernel<CC, VV, MODE><<<dim3(GX, H, dv / VS), CTHREADS, lds, stream>>>(proj, row_w, bias_i, bias_f, work, dens, \
        cu_seqlens, slots, S, n, m, H, d, dv, cap, ws);                                                              \
  } while (0)
#define GO(MODE, GX)                                      \
  do {                                                    \
    if (C == 64 && VS == 64) GO_MODE(64, 64, MODE, GX);   \
    else if (C == 64 && VS == 32) GO_MODE(64, 32, MODE, GX); \
    else if (C == 64) GO_MODE(64, 16, MODE, GX);          \
    else if (VS == 32) GO_MODE(32, 32, MODE, GX);         \
    else GO_MODE(32, 16, MODE, GX);                       \
  } while (0)
  if (!side_by_side) {
    GO(0, n_seqs);
  } else {
    GO(1, n_seqs * ws.max_chunks);
    ALICE_LAUNCH_CHECK();
    mlstm_chunk_states_kernel<<<dim3(n_seqs, H, ceil_div((long)d * dv / 4, THREADS)), THREADS, 0, stream>>>(
        cu_seqlens, slots, S, n, m, H, d, dv, C, ws);
    ALICE_LAUNCH_CHECK();
    GO(2, n_seqs * ws.max_chunks);
  }
#undef GO
#undef GO_MODE
  ALICE_LAUNCH_CHECK();
  const int threads = dv >= 256 ? 256 : (dv >= 128 ? 128 : 64);
  if (out_dtype == DT_F32)
    mlstm_finish_kernel<float><<<dim3(T, H), threads, 0, stream>>>(work, dens, proj, row_w, norm_w, norm_dtype, (float*)out, H, d, dv, eps);
  else
    mlstm_finish_kernel<bf16_t><<<dim3(T, H), threads, 0, stream>>>(work, dens, proj, row_w, norm_w, norm_dtype, (bf16_t*)out, H, d, dv, eps);
  ALICE_LAUNCH_CHECK();
  return 0;
}
