// Attention over the paged cache for any head size up to 256, any head and group counts, in
// 32-bit arithmetic: the kernel of the true 32-bit path and the fallback of the bfloat16 path.
// One block per (query token, query head); used for prompts and for single decoded tokens alike.
//
// Order of operations as in the reference (llama3.rs:5622-5688): dot product, times scale, softcap
// cap * tanh(s / cap), then the softmax over the keys max(0, pos + 1 - window) .. pos (window keys,
// the query's own included, llama3.rs:5444-5451), then the weighted sum of the values; the kv head
// of query head h is h / (nH / nKV).  The softmax is computed chunk by chunk with a running maximum
// (the reference's online variant, llama3.rs:5568-5620).  A position term at the score stage is a
// parameter: with bias_slopes, head h's capped score of key k for the query at position p gets
// bias_slopes[h] * (k - p) added (a linear distance bias; the reference's models have none, so the
// product passes a null pointer).
//
// Further parameters of the mask and the softmax (AttnExtras; all off for the product's architecture):
// chunk: the query at position p sees the keys of its own chunk only, floor(k / chunk) == floor(p / chunk),
// chunks counted from position 0; keep_first: beside its window a query also sees the keys k < keep_first,
// at their true positions; sink: one number a head whose exponential joins the softmax's denominator and
// has no value; vrot_cos / vrot_sin: the values were cached rotated by their positions (pairs (2m, 2m + 1),
// tables [positions, dv / 2]) and the head's output is turned back by the query's position; gate_mode 2: the
// gate is one number an output element, [T, nH * dv]; value_heads > 0: every query head's weights are applied
// to the values of each of the nKV value heads in turn (blockIdx.z), and the float32 results
// [T, nH, nKV, dv] go to out32 (for a mix of the heads' weights behind this kernel); gate32: the gate as
// float32 rows; out_scale: a constant factor of the gated output.
#include "common.h"
#include "alice_hip.h"

namespace {

constexpr int CHUNK = 1024;
constexpr int THREADS = 256;

struct AttnExtras {
  int chunk, keep_first, gate_mode, value_heads;
  const float* sink;
  const float* vrot_cos;
  const float* vrot_sin;
  float* out32;
  const float* gate32;      // the gate in float32 (rows of a float32 projection), read in place of `gate`
  int gate32_stride;
  float out_scale;          // a constant factor of the output
};

template <typename T, bool FULL>
__global__ __launch_bounds__(THREADS) void attn_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_pool, const T* __restrict__ v_pool, T* __restrict__ out,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ block_table, int bt_stride, int nH, int nKV, int d, int page_size,
    float scale, float cap, int window, int DG, const float* __restrict__ bias_slopes,
    int dv, const T* __restrict__ gate, int gate_stride, AttnExtras x) {
  __shared__ float qs[256];
  __shared__ float sc[CHUNK];
  __shared__ float red[17];
  __shared__ float part[THREADS];

  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int pos = positions[t];
  const int seq = seq_of_token[t];
  const int kvh = h / (nH / nKV);
  const float slope = bias_slopes ? bias_slopes[h] : 0.f;
  const int start = x.chunk > 0 ? (pos / x.chunk) * x.chunk : (window > 0 ? max(0, pos + 1 - window) : 0);
  // the visible keys: the first n_first positions (kept beside the window), then start .. pos
  const int n_first = x.keep_first > 0 ? min(x.keep_first, start) : 0;
  const int n_keys = n_first + pos + 1 - start;
  const int vh = x.value_heads > 0 ? (int)blockIdx.z : kvh;
  const int* bt = block_table + (size_t)seq * bt_stride;

  const T* qrow = q + ((size_t)t * nH + h) * d;
  for (int i = tid; i < d; i += THREADS) qs[i] = load_f32(qrow, i);
  __syncthreads();

  const int G = THREADS / DG;            // key groups in the value pass
  const int g = tid / DG, j = tid % DG;
  float acc = 0.f, m_run = -INFINITY, l_run = 0.f;

  for (int c0 = 0; c0 < n_keys; c0 += CHUNK) {
    const int n = min(CHUNK, n_keys - c0);
    float lmax = -INFINITY;
    for (int i = tid; i < n; i += THREADS) {
      const int kp = c0 + i < n_first ? c0 + i : start + (c0 + i - n_first);
      const int page = bt[kp / page_size];
      const T* krow = k_pool + (((size_t)page * nKV + kvh) * page_size + kp % page_size) * d;
      float s = 0.f;
      for (int e = 0; e < d; ++e) s = fmaf(qs[e], load_f32(krow, e), s);
      s *= scale;
      if (cap > 0.f) s = cap * (FULL ? tanh_full(s / cap) : tanh_fast(s / cap));
      if (bias_slopes) s = fmaf(slope, (float)(kp - pos), s);
      sc[i] = s;
      lmax = fmaxf(lmax, s);
    }
    const float m_new = fmaxf(m_run, block_max(lmax, red));
    const float corr = (m_run == -INFINITY) ? 0.f : (FULL ? expf(m_run - m_new) : __expf(m_run - m_new));
    float lsum = 0.f;
    for (int i = tid; i < n; i += THREADS) {
      float p = FULL ? expf(sc[i] - m_new) : __expf(sc[i] - m_new);
      sc[i] = p;
      lsum += p;
    }
    l_run = l_run * corr + block_sum(lsum, red);      // the barriers inside also publish sc[]
    m_run = m_new;
    acc *= corr;
    if (j < dv) {
      for (int i = g; i < n; i += G) {
        const int kp = c0 + i < n_first ? c0 + i : start + (c0 + i - n_first);
        const int page = bt[kp / page_size];
        const T* vrow = v_pool + (((size_t)page * nKV + vh) * page_size + kp % page_size) * dv;
        acc = fmaf(sc[i], load_f32(vrow, j), acc);
      }
    }
    __syncthreads();                                   // sc[] is rewritten by the next chunk
  }
  part[tid] = acc;
  __syncthreads();
  if (x.sink) {                                       // one more term of the denominator, without a value
    const float sk = x.sink[h];
    const float m_fin = fmaxf(m_run, sk);
    const float corr = FULL ? expf(m_run - m_fin) : __expf(m_run - m_fin);
    l_run = l_run * corr + (FULL ? expf(sk - m_fin) : __expf(sk - m_fin));
    acc = corr;                                        // reused below as the outputs' factor
  } else {
    acc = 1.f;
  }
  float o = 0.f;
  if (tid < dv) {
    for (int gg = 0; gg < G; ++gg) o += part[gg * DG + tid];
    o = o * acc / l_run;
  }
  if (x.vrot_cos) {                                   // turn the output back by the query's position
    __syncthreads();
    part[tid] = o;
    __syncthreads();
    if (tid < dv) {
      const int m = tid >> 1;
      const float c = x.vrot_cos[(size_t)pos * (dv >> 1) + m], s = x.vrot_sin[(size_t)pos * (dv >> 1) + m];
      // the pair (u, v) turned by -angle: (u c + v s, v c - u s)
      o = (tid & 1) ? fmaf(part[tid], c, -__fmul_rn(part[tid - 1], s)) : fmaf(part[tid], c, __fmul_rn(part[tid + 1], s));
    }
  }
  if (tid < dv) {
    if (x.value_heads > 0) {
      x.out32[(((size_t)t * nH + h) * nKV + vh) * dv + tid] = o;
      return;
    }
    if (x.gate32) o *= sigmoid_f(x.gate32[(size_t)t * x.gate32_stride + (x.gate_mode == 2 ? h * dv + tid : h)], FULL);
    else if (gate) o *= sigmoid_f(load_f32(gate, (size_t)t * gate_stride + h), FULL);
    o *= x.out_scale;
    store_f32(out + ((size_t)t * nH + h) * dv, tid, o);
  }
}

// out[t, h, e] = sigmoid(gate[t, h dv + e]) * sum_g talk[h, g] * a[t, g, kv head of h, e]: the heads' softmax
// weights mixed by talk [nH, nH], each head applying its mixed weights to its own kv head's values, written
// as a mix of the per-(head, value head) outputs that the attention kernel left in a (float32).
template <typename T, bool FULL>
__global__ void mix_heads_kernel(const float* __restrict__ a, const float* __restrict__ talk, const float* __restrict__ gate,
                                 int gate_stride, float out_scale, T* __restrict__ out, int nH, int nKV, int dv) {
  const int t = blockIdx.x, h = blockIdx.y;            // a block per (token, head)
  const int c = h / (nH / nKV);
  for (int e = threadIdx.x; e < dv; e += blockDim.x) {
    float o = 0.f;
    for (int g = 0; g < nH; ++g) o = fmaf(talk[h * nH + g], a[(((size_t)t * nH + g) * nKV + c) * dv + e], o);
    if (gate) o *= sigmoid_f(gate[(size_t)t * gate_stride + h * dv + e], FULL);
    store_f32(out + ((size_t)t * nH + h) * dv, e, o * out_scale);
  }
}

// The same with a block per (token, kv head): the kv head's column of all heads' outputs goes through LDS once and
// serves the group's heads (dynamic LDS of nH * dv floats).
template <typename T, bool FULL>
__global__ void mix_heads_group_kernel(const float* __restrict__ a, const float* __restrict__ talk, const float* __restrict__ gate,
                                       int gate_stride, float out_scale, T* __restrict__ out, int nH, int nKV, int dv) {
  extern __shared__ float col[];                       // [nH][dv]
  const int t = blockIdx.x, c = blockIdx.y, per = nH / nKV;
  for (int i = threadIdx.x; i < nH * dv; i += blockDim.x)
    col[i] = a[(((size_t)t * nH + i / dv) * nKV + c) * dv + i % dv];
  __syncthreads();
  for (int i = threadIdx.x; i < per * dv; i += blockDim.x) {
    const int h = c * per + i / dv, e = i % dv;
    float o = 0.f;
    for (int g = 0; g < nH; ++g) o = fmaf(talk[h * nH + g], col[g * dv + e], o);
    if (gate) o *= sigmoid_f(gate[(size_t)t * gate_stride + h * dv + e], FULL);
    store_f32(out + ((size_t)t * nH + h) * dv, e, o * out_scale);
  }
}

}  // namespace

static int attention_generic_launch(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out,
                                    const int* positions, const int* seq_of_token, const int* block_table,
                                    int bt_stride, int T, int nH, int nKV, int d, int page_size, float scale,
                                    float softcap, int window, const float* bias_slopes, int full_precision,
                                    int dv, const void* gate, int gate_stride, AttnExtras x, hipStream_t stream) {
  if (dv <= 0) dv = d;
  ALICE_CHECK(gate == nullptr || gate_stride >= nH, "attention: gate rows of %d elements are too short for %d heads", gate_stride, nH);
  ALICE_CHECK(x.gate32 == nullptr || x.gate32_stride >= (x.gate_mode == 2 ? nH * dv : nH), "attention: gate rows of %d elements are too short", x.gate32_stride);
  ALICE_CHECK(dtype_ok(dtype), "attention: unknown dtype %d", dtype);
  ALICE_CHECK(T >= 0 && nH >= 1 && nKV >= 1 && nH % nKV == 0, "attention: bad head counts nH=%d nKV=%d", nH, nKV);
  ALICE_CHECK(d >= 1 && d <= 256, "attention: head_dim %d is outside 1..256, the range of this kernel", d);
  ALICE_CHECK(dv <= 256, "attention: value head size %d is outside 1..256, the range of this kernel", dv);
  ALICE_CHECK(nH <= 65535 && nKV <= 65535, "attention: too many heads for one launch (%d)", nH);
  ALICE_CHECK(page_size > 0 && bt_stride > 0, "attention: bad page geometry");
  ALICE_CHECK(softcap >= 0.f && window >= 0, "attention: softcap and window must not be negative (0 turns them off)");
  ALICE_CHECK(x.chunk >= 0 && x.keep_first >= 0, "attention: chunk and keep_first must not be negative (0 turns them off)");
  ALICE_CHECK((x.vrot_cos == nullptr) == (x.vrot_sin == nullptr) && (x.vrot_cos == nullptr || dv % 2 == 0),
              "attention: turning the output back needs both tables and an even value head size");
  ALICE_CHECK(x.value_heads == 0 || (x.value_heads == nKV && x.out32 != nullptr), "attention: per-value-head outputs need their float32 buffer");
  if (T == 0) return 0;
  int DG = 1;
  while (DG < dv) DG <<= 1;
  dim3 grid(T, nH, x.value_heads > 0 ? nKV : 1);
  DISPATCH_DTYPE(dtype, TT, {
    if (full_precision)
      attn_generic_kernel<TT, true><<<grid, THREADS, 0, stream>>>((const TT*)q, (const TT*)k_pool, (const TT*)v_pool,
          (TT*)out, positions, seq_of_token, block_table, bt_stride, nH, nKV, d, page_size, scale, softcap, window, DG, bias_slopes, dv, (const TT*)gate, gate_stride, x);
    else
      attn_generic_kernel<TT, false><<<grid, THREADS, 0, stream>>>((const TT*)q, (const TT*)k_pool, (const TT*)v_pool,
          (TT*)out, positions, seq_of_token, block_table, bt_stride, nH, nKV, d, page_size, scale, softcap, window, DG, bias_slopes, dv, (const TT*)gate, gate_stride, x);
  });
  ALICE_LAUNCH_CHECK();
  return 0;
}

extern "C" int alice_attention_generic(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out,
                                       const int* positions, const int* seq_of_token, const int* block_table,
                                       int bt_stride, int T, int nH, int nKV, int d, int page_size, float scale,
                                       float softcap, int window, const float* bias_slopes, int full_precision,
                                       int dv, const void* gate, int gate_stride, hipStream_t stream) {
  AttnExtras x{0, 0, 1, 0, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 1.f};
  return attention_generic_launch(q, dtype, k_pool, v_pool, out, positions, seq_of_token, block_table, bt_stride, T, nH, nKV,
                                  d, page_size, scale, softcap, window, bias_slopes, full_precision, dv, gate, gate_stride, x, stream);
}

extern "C" int alice_attention_masked(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out,
                                      const int* positions, const int* seq_of_token, const int* block_table,
                                      int bt_stride, int T, int nH, int nKV, int d, int page_size, float scale,
                                      float softcap, int window, const float* bias_slopes, int full_precision,
                                      int dv, const float* gate, int gate_stride, int gate_mode, float out_scale, int chunk,
                                      int keep_first, const float* sink, const float* vrot_cos, const float* vrot_sin,
                                      float* out32, hipStream_t stream) {
  ALICE_CHECK(gate_mode == 1 || gate_mode == 2, "attention: gate mode %d is not known (1: a number a head, 2: a number an element)", gate_mode);
  AttnExtras x{chunk, keep_first, gate_mode, out32 ? nKV : 0, sink, vrot_cos, vrot_sin, out32, gate, gate_stride, out_scale};
  return attention_generic_launch(q, dtype, k_pool, v_pool, out, positions, seq_of_token, block_table, bt_stride, T, nH, nKV,
                                  d, page_size, scale, softcap, window, bias_slopes, full_precision, dv, nullptr, 0, x, stream);
}

extern "C" int alice_mix_heads(const float* a, const float* talk, const float* gate, int gate_stride, float out_scale, void* out,
                               int dtype, int T, int nH, int nKV, int dv, int full_precision, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(dtype), "mix_heads: unknown dtype %d", dtype);
  ALICE_CHECK(a && talk && out && T >= 0 && nH >= 1 && nH <= 65535 && nKV >= 1 && nH % nKV == 0 && dv >= 1, "mix_heads: bad arguments");
  ALICE_CHECK(gate == nullptr || gate_stride >= nH * dv, "mix_heads: gate rows of %d elements are too short", gate_stride);
  if (T == 0) return 0;
  if ((size_t)nH * dv * sizeof(float) <= 48 * 1024 && nKV <= 65535) {      // the column fits LDS: a block per (token, kv head)
    const size_t lds = (size_t)nH * dv * sizeof(float);
    DISPATCH_DTYPE(dtype, TT, {
      if (full_precision) mix_heads_group_kernel<TT, true><<<dim3(T, nKV), 256, lds, stream>>>(a, talk, gate, gate_stride, out_scale, (TT*)out, nH, nKV, dv);
      else mix_heads_group_kernel<TT, false><<<dim3(T, nKV), 256, lds, stream>>>(a, talk, gate, gate_stride, out_scale, (TT*)out, nH, nKV, dv);
    });
    ALICE_LAUNCH_CHECK();
    return 0;
  }
  DISPATCH_DTYPE(dtype, TT, {
    if (full_precision) mix_heads_kernel<TT, true><<<dim3(T, nH), dv > 128 ? 256 : (dv > 64 ? 128 : 64), 0, stream>>>(a, talk, gate, gate_stride, out_scale, (TT*)out, nH, nKV, dv);
    else mix_heads_kernel<TT, false><<<dim3(T, nH), dv > 128 ? 256 : (dv > 64 ? 128 : 64), 0, stream>>>(a, talk, gate, gate_stride, out_scale, (TT*)out, nH, nKV, dv);
  });
  ALICE_LAUNCH_CHECK();
  return 0;
}
