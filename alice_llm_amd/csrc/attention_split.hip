// Attention of single tokens over a row-major paged cache with the masks and softmax terms of
// alice_attention_masked, the keys split over blocks: 32-bit arithmetic on operands of either dtype (the decode kernel
// of the mixers that the matrix-core decode kernel does not take, and of the true 32-bit path).
//
// A block takes one token, one kv head and one run of 256 visible keys, a thread one key: it has the whole key row
// on its way from memory at once (16-byte loads), and scores it against every query head of the kv head's group,
// whose queries lie in LDS; the key row is read once for the group.  The block's maximum and sum a head come from
// two barriers; then the threads turn to the values: a thread owns 16 bytes of the value row's width for a share of
// the keys, with one accumulator set a head, the shares meet by lane swaps and through LDS.  With per-value-head
// outputs the second phase runs once for every kv head's values.  Each block leaves (maximum, sum, unnormalised
// output) per head; attn_split_combine_kernel merges the runs in their order, adds the sink to the denominator,
// turns the output back where the values were cached turned, applies gate and factor, and writes the result (or
// the per-value-head outputs in float32 for the mix of the heads that follows).
#include "common.h"
#include "alice_hip.h"

namespace {

constexpr int KEYS = 256;

struct SplitArgs {
  const int* positions;
  const int* seq_of_token;
  const int* block_table;
  int bt_stride, nH, nKV, d, dv, page_size;
  float scale;
  int window, chunk, keep_first, n_splits, value_heads;
  const float* slopes;
  float* part_ml;      // [T, nH, splits, 2]
  float* part_o;       // [T, nH, value heads (or 1), splits, dv]
};

template <typename T> __device__ __forceinline__ void unpack16(const uint4& w, float* f);
template <> __device__ __forceinline__ void unpack16<float>(const uint4& w, float* f) {
  f[0] = __uint_as_float(w.x); f[1] = __uint_as_float(w.y); f[2] = __uint_as_float(w.z); f[3] = __uint_as_float(w.w);
}
template <> __device__ __forceinline__ void unpack16<bf16_t>(const uint4& w, float* f) {
  const uint32_t v[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = bf16_bits_to_f32(v[i] & 0xffffu);
    f[2 * i + 1] = bf16_bits_to_f32(v[i] >> 16);
  }
}

template <typename T, int PER>
__global__ __launch_bounds__(256) void attn_split_kernel(const T* __restrict__ q, const T* __restrict__ k_pool,
                                                         const T* __restrict__ v_pool, SplitArgs a) {
  constexpr bool FULL = sizeof(T) == 4;
  constexpr int VEC = 16 / sizeof(T);
  __shared__ __align__(16) float qs[PER][256];
  __shared__ float ps[PER][KEYS];
  __shared__ int rows_of[KEYS];                       // the row of each of the block's keys in kv head 0's part of its page
  __shared__ float wred[4][PER];
  __shared__ __align__(16) float ored[4][256];

  const int t = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int d = a.d, dv = a.dv, per = a.nH / a.nKV, h0 = kvh * per;
  const int pos = a.positions[t];
  const int* bt = a.block_table + (size_t)a.seq_of_token[t] * a.bt_stride;
  const int start = a.chunk > 0 ? (pos / a.chunk) * a.chunk : (a.window > 0 ? max(0, pos + 1 - a.window) : 0);
  const int n_first = (a.keep_first > 0 && a.window > 0 && a.chunk == 0) ? min(a.keep_first, start) : 0;
  const int n_keys = n_first + pos + 1 - start;
  const int v0 = split * KEYS, nk = max(0, min(KEYS, n_keys - v0));

  // the group's queries (rows beyond the group stay zero)
  for (int i = tid; i < PER * d; i += 256) {
    const int hh = i / d, e = i % d;
    qs[hh][e] = hh < per ? load_f32(q + ((size_t)t * a.nH + h0 + hh) * d, e) : 0.f;
  }
  // this thread's key
  const bool has = tid < nk;
  const int vi = v0 + tid;
  const int kp = has ? (vi < n_first ? vi : start + (vi - n_first)) : 0;
  const int row0 = has ? bt[kp / a.page_size] * a.nKV * a.page_size + kp % a.page_size : 0;
  rows_of[tid] = row0;
  __syncthreads();
  float dot[PER];
#pragma unroll
  for (int hh = 0; hh < PER; ++hh) dot[hh] = 0.f;
  if (has) {
    const T* krow = k_pool + ((size_t)row0 + (size_t)kvh * a.page_size) * d;
    for (int c0 = 0; c0 < d; c0 += 8 * VEC) {           // eight loads on their way at a time
      uint4 w[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (c0 + j * VEC < d) w[j] = *reinterpret_cast<const uint4*>(krow + c0 + j * VEC);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (c0 + j * VEC >= d) break;
        float kf[VEC];
        unpack16<T>(w[j], kf);
#pragma unroll
        for (int i = 0; i < VEC; i += 4) {
#pragma unroll
          for (int hh = 0; hh < PER; ++hh) {
            const float4 qq = *reinterpret_cast<const float4*>(&qs[hh][c0 + j * VEC + i]);
            dot[hh] = fmaf(qq.x, kf[i], dot[hh]);
            dot[hh] = fmaf(qq.y, kf[i + 1], dot[hh]);
            dot[hh] = fmaf(qq.z, kf[i + 2], dot[hh]);
            dot[hh] = fmaf(qq.w, kf[i + 3], dot[hh]);
          }
        }
      }
    }
  }
  // scores, the block's maximum a head, the weights and their sum
  float sc[PER];
#pragma unroll
  for (int hh = 0; hh < PER; ++hh) {
    float s = dot[hh] * a.scale;
    if (a.slopes && hh < per) s = fmaf(a.slopes[h0 + hh], (float)(kp - pos), s);
    sc[hh] = has ? s : -INFINITY;
    const float m = wave_max(sc[hh]);
    if (lane == 0) wred[wave][hh] = m;
  }
  __syncthreads();
  float mx[PER];
#pragma unroll
  for (int hh = 0; hh < PER; ++hh) mx[hh] = fmaxf(fmaxf(wred[0][hh], wred[1][hh]), fmaxf(wred[2][hh], wred[3][hh]));
  __syncthreads();
#pragma unroll
  for (int hh = 0; hh < PER; ++hh) {
    const float p = has ? (FULL ? expf(sc[hh] - mx[hh]) : __expf(sc[hh] - mx[hh])) : 0.f;
    ps[hh][tid] = p;
    const float s = wave_sum(p);
    if (lane == 0) wred[wave][hh] = s;
  }
  __syncthreads();
#pragma unroll
  for (int hh = 0; hh < PER; ++hh) {
    if (tid == hh && hh < per) {
      float* ml = a.part_ml + (((size_t)t * a.nH + h0 + hh) * a.n_splits + split) * 2;
      ml[0] = mx[hh];
      ml[1] = (wred[0][hh] + wred[1][hh]) + (wred[2][hh] + wred[3][hh]);
    }
  }
  // values: thread (kg, ec) takes the keys kg, kg + KG, .. and 16 bytes of the row's width
  const int EC = dv / VEC;
  int EC2 = 1;
  while (EC2 < EC) EC2 <<= 1;
  const int KG = 256 / EC2, ec = tid % EC2, kg = tid / EC2;
  const int n_vh = a.value_heads > 0 ? a.value_heads : 1;
  for (int z = 0; z < n_vh; ++z) {
    const int vh = a.value_heads > 0 ? z : kvh;
    float acc[PER][VEC];
#pragma unroll
    for (int hh = 0; hh < PER; ++hh)
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[hh][i] = 0.f;
    if (ec < EC) {
      for (int i = kg; i < nk; i += KG) {
        const uint4 w = *reinterpret_cast<const uint4*>(v_pool + ((size_t)rows_of[i] + (size_t)vh * a.page_size) * dv + ec * VEC);
        float vf[VEC];
        unpack16<T>(w, vf);
#pragma unroll
        for (int hh = 0; hh < PER; ++hh) {
          const float p = ps[hh][i];
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[hh][e] = fmaf(p, vf[e], acc[hh][e]);
        }
      }
    }
    // the shares of the keys meet: lane swaps within a wave, then the four waves through LDS, a head at a time
#pragma unroll
    for (int hh = 0; hh < PER; ++hh) {
      if (hh >= per) break;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float v = acc[hh][e];
        for (int off = EC2; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
        acc[hh][e] = v;
      }
      __syncthreads();                                    // ored is free again
      if (EC2 >= 64) {                                    // a wave holds one share only: the waves hold KG = 4 / (EC2 / 64) shares
        if (ec < EC)
#pragma unroll
          for (int e = 0; e < VEC; ++e) ored[kg % 4][(size_t)ec * VEC + e] = (kg < 4) ? acc[hh][e] : 0.f;
      } else if (lane < EC2 && ec < EC) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) ored[wave][ec * VEC + e] = acc[hh][e];
      }
      __syncthreads();
      const int shares = EC2 >= 64 ? KG : 4;
      float* po = a.part_o + ((((size_t)t * a.nH + h0 + hh) * n_vh + z) * a.n_splits + split) * dv;
      for (int e = tid; e < dv; e += 256) {
        float o = 0.f;
        for (int s = 0; s < shares; ++s) o += ored[s][e];
        po[e] = o;
      }
    }
  }
}

struct CombineArgs {
  const int* positions;
  int nH, nKV, dv, n_splits, value_heads;
  const float* part_ml;
  const float* part_o;
  const float* sink;
  const float* vcos;
  const float* vsin;
  const float* gate;
  int gate_stride, gate_mode;
  float out_scale;
  float* out32;
};

template <typename T>
__global__ void attn_split_combine_kernel(T* __restrict__ out, CombineArgs a) {
  constexpr bool FULL = sizeof(T) == 4;
  const int t = blockIdx.x, h = blockIdx.y, z = blockIdx.z, dv = a.dv, S = a.n_splits;
  const int n_vh = a.value_heads > 0 ? a.value_heads : 1;
  const float* ml = a.part_ml + ((size_t)t * a.nH + h) * S * 2;
  float M = -INFINITY;
  for (int s = 0; s < S; ++s) M = fmaxf(M, ml[2 * s]);
  const float sk = a.sink ? a.sink[h] : -INFINITY;
  const float Mf = fmaxf(M, sk);
  float L = a.sink ? (FULL ? expf(sk - Mf) : __expf(sk - Mf)) : 0.f;
  for (int s = 0; s < S; ++s) {
    const float w = ml[2 * s] > -INFINITY ? (FULL ? expf(ml[2 * s] - Mf) : __expf(ml[2 * s] - Mf)) : 0.f;
    L = fmaf(ml[2 * s + 1], w, L);
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  const float* po = a.part_o + (((size_t)t * a.nH + h) * n_vh + z) * S * dv;
  const int pos = a.positions[t];
  for (int m = threadIdx.x; 2 * m < dv; m += blockDim.x) {            // the pair (2m, 2m + 1); a last odd element alone
    const bool two = 2 * m + 1 < dv;
    float o0 = 0.f, o1 = 0.f;
    for (int s = 0; s < S; ++s) {
      const float w = ml[2 * s] > -INFINITY ? (FULL ? expf(ml[2 * s] - Mf) : __expf(ml[2 * s] - Mf)) : 0.f;
      o0 = fmaf(po[(size_t)s * dv + 2 * m], w, o0);
      if (two) o1 = fmaf(po[(size_t)s * dv + 2 * m + 1], w, o1);
    }
    o0 *= inv;
    o1 *= inv;
    if (a.vcos) {
      const float c = a.vcos[(size_t)pos * (dv >> 1) + m], sn = a.vsin[(size_t)pos * (dv >> 1) + m];
      const float u = o0, v = o1;
      o0 = fmaf(u, c, __fmul_rn(v, sn));
      o1 = fmaf(v, c, -__fmul_rn(u, sn));
    }
    if (a.out32) {
      float* dst = a.out32 + (((size_t)t * a.nH + h) * a.nKV + z) * dv;
      dst[2 * m] = o0;
      if (two) dst[2 * m + 1] = o1;
      continue;
    }
    if (a.gate) {
      const float* g = a.gate + (size_t)t * a.gate_stride;
      o0 *= sigmoid_f(a.gate_mode == 2 ? g[h * dv + 2 * m] : g[h], FULL);
      if (two) o1 *= sigmoid_f(a.gate_mode == 2 ? g[h * dv + 2 * m + 1] : g[h], FULL);
    }
    T* dst = out + ((size_t)t * a.nH + h) * dv;
    store_f32(dst, 2 * m, o0 * a.out_scale);
    if (two) store_f32(dst, 2 * m + 1, o1 * a.out_scale);
  }
}

}  // namespace

extern "C" int alice_attention_split_supported(int dtype, int nH, int nKV, int d, int dv) {
  const int vec = dtype == DT_F32 ? 4 : 8;
  return nKV >= 1 && nH % nKV == 0 && nH / nKV <= 16 && d >= vec && dv >= vec && d % vec == 0 && dv % vec == 0 && d <= 256 && dv <= 256;
}

// The number of key runs for at most max_keys visible keys a token, and the float32 workspace for T tokens.
extern "C" int alice_attention_split_runs(int max_keys) { return max(1, ceil_div(max_keys, KEYS)); }
extern "C" long alice_attention_split_workspace(int T, int nH, int nKV, int dv, int runs, int per_value_head) {
  return (long)T * nH * runs * 2 + (long)T * nH * (per_value_head ? nKV : 1) * runs * dv;
}

// alice_attention_masked's result by the key-split kernels; max_keys: the most keys any token of the step sees (the
// caller knows it from the step's longest context and the mask); work: alice_attention_split_workspace floats.
extern "C" int alice_attention_split(const void* q, int dtype, const void* k_pool, const void* v_pool, void* out, float* out32,
                                     const int* positions, const int* seq_of_token, const int* block_table, int bt_stride,
                                     int T, int nH, int nKV, int d, int dv, int page_size, float scale, int window, int chunk,
                                     int keep_first, int max_keys, const float* bias_slopes, const float* sink,
                                     const float* vrot_cos, const float* vrot_sin, const float* gate, int gate_stride,
                                     int gate_mode, float out_scale, float* work, hipStream_t stream) {
  ALICE_CHECK(dtype_ok(dtype), "attention: unknown dtype %d", dtype);
  ALICE_CHECK(alice_attention_split_supported(dtype, nH, nKV, d, dv), "attention: heads %d / %d of sizes %d and %d are outside this kernel's range", nH, nKV, d, dv);
  ALICE_CHECK(q && k_pool && v_pool && (out || out32) && positions && seq_of_token && block_table && work, "attention: a pointer is missing");
  ALICE_CHECK(T >= 0 && page_size > 0 && bt_stride > 0 && max_keys >= 1, "attention: bad sizes");
  ALICE_CHECK(window >= 0 && chunk >= 0 && keep_first >= 0, "attention: window, chunk and keep_first must not be negative (0 turns them off)");
  ALICE_CHECK((vrot_cos == nullptr) == (vrot_sin == nullptr) && (vrot_cos == nullptr || dv % 2 == 0), "attention: turning the output back needs both tables and an even value head size");
  ALICE_CHECK(gate == nullptr || (gate_mode == 1 && gate_stride >= nH) || (gate_mode == 2 && gate_stride >= nH * dv),
              "attention: gate rows of %d elements are too short", gate_stride);
  ALICE_CHECK(((uintptr_t)q & 15) == 0 && ((uintptr_t)k_pool & 15) == 0 && ((uintptr_t)v_pool & 15) == 0, "attention: operands are not aligned");
  if (T == 0) return 0;
  const int runs = alice_attention_split_runs(max_keys);
  ALICE_CHECK(runs <= 65535 && nKV <= 65535 && nH <= 65535, "attention: too many heads or keys for one launch");
  const int n_vh = out32 ? nKV : 0;
  float* part_ml = work;
  float* part_o = work + (size_t)T * nH * runs * 2;
  SplitArgs a{positions, seq_of_token, block_table, bt_stride, nH, nKV, d, dv, page_size, scale, window, chunk, keep_first, runs, n_vh,
              bias_slopes, part_ml, part_o};
  const int per = nH / nKV;
  dim3 grid(T, nKV, runs);
#define GO(TT, PER) attn_split_kernel<TT, PER><<<grid, 256, 0, stream>>>((const TT*)q, (const TT*)k_pool, (const TT*)v_pool, a)
#define BY_PER(TT)                 \
  do {                             \
    if (per <= 1) GO(TT, 1);       \
    else if (per <= 2) GO(TT, 2);  \
    else if (per <= 4) GO(TT, 4);  \
    else if (per <= 8) GO(TT, 8);  \
    else GO(TT, 16);               \
  } while (0)
  if (dtype == DT_F32) BY_PER(float);
  else BY_PER(bf16_t);
#undef BY_PER
#undef GO
  ALICE_LAUNCH_CHECK();
  CombineArgs c{positions, nH, nKV, dv, runs, n_vh, part_ml, part_o, sink, vrot_cos, vrot_sin, gate, gate_stride, gate_mode, out_scale, out32};
  dim3 g2(T, nH, out32 ? nKV : 1);
  const int threads = dv > 128 ? 128 : 64;
  if (dtype == DT_F32) attn_split_combine_kernel<float><<<g2, threads, 0, stream>>>((float*)out, c);
  else attn_split_combine_kernel<bf16_t><<<g2, threads, 0, stream>>>((bf16_t*)out, c);
  ALICE_LAUNCH_CHECK();
  return 0;
}
