// Prompt attention on the matrix cores over a row-major paged cache, with the masks and softmax terms of
// alice_attention_masked: a window with kept first positions, chunks, a linear distance term, a sink, values that
// were cached turned by their position (the output is turned back), a gate an element or a head, a constant factor,
// and the per-value-head outputs that a mix of the heads' weights needs.  bfloat16 operands, 32-bit scores, softmax
// and sums.
//
// A block of four waves takes 64 consecutive queries of one sequence and HPW query heads of one kv head's group
// (1; 2 or 4 at the caller's wish), a wave 16 of the queries for all of those heads: a staged block of keys and
// values, and every fragment a wave reads of it, serves all of them.  The
// keys go through LDS 32 at a time, in two buffers (the next 32 are on their way from memory while the waves work
// on the current ones, their page number looked up a step further ahead, and one barrier a step suffices): the key rows as they are, the value rows transposed.  A wave computes the transposed score tile S^T = K Q^T with v_mfma_f32_16x16x32_bf16
// (keys are the rows, the wave's 16 queries the columns), so that a lane holds eight scores of ONE query: the
// softmax's maximum and sum are four-lane affairs, and the rounded weights are, as they stand, the second operand
// of O^T = V^T P^T; the transposed values lie in LDS in the key order in which the score tiles leave the matrix
// instruction (keys g*4 .. g*4+3 and 16 + g*4 .. for lane group g).  Key blocks that no query of the block can see
// are not visited (the kept first positions are a second run of blocks), and a wave skips the second product
// for a block none of whose keys its queries see.  Head sizes are padded with zeros to 64, 128 or 256.
#include "common.h"
#include "alice_hip.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mfma32(u32x4 a, u32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

struct TiledArgs {
  const bf16_t* q;
  const bf16_t* k_pool;
  const bf16_t* v_pool;
  bf16_t* out;
  float* out32;
  const int* positions;
  const int* cu_seqlens;
  const int* block_table;
  int bt_stride, n_seqs, nH, nKV, d, dv, page_size;
  float scale;
  int window, chunk, keep_first, page_shift;     // page_shift: log2 of the page size, or -1 where that is no power of two
  const float* slopes;
  const float* sink;
  const float* vcos;
  const float* vsin;
  const float* gate;
  int gate_stride, gate_mode;
  float out_scale;
};

constexpr int KT = 32;        // keys a step
constexpr int VPAD = 40;      // row length of the transposed values in LDS (32 keys and a pad against bank conflicts)

template <int DP, int DVP, int HPW>
__global__ __launch_bounds__(256) void attn_tiled_kernel(TiledArgs a) {
  constexpr int KS = DP / 32, ET = DVP / 16;
  constexpr int KROW = DP + 8;
  constexpr int NKC = DP / 64, NVC = DVP / 64;          // 16-byte pieces of keys / values a thread moves a step
  constexpr int NBUF = (DP + DVP <= 384) ? 2 : 1;        // two buffers where they fit the static LDS limit
  __shared__ __align__(16) bf16_t Ks[NBUF][KT][KROW];
  __shared__ __align__(16) bf16_t Vt[NBUF][DVP][VPAD];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, g = lane >> 4;
  const int h0 = blockIdx.y * HPW;                      // the wave's heads: h0 .. h0 + HPW - 1, of one kv head
  const int per = a.nH / a.nKV, kvh = h0 / per;
  const int vh = a.out32 ? (int)blockIdx.z : kvh;
  const int D = a.d, DV = a.dv;

  // which 64 queries: the blocks are dealt to the sequences in order, ceil(tokens / 64) each; the hardware starts
  // blocks in the order of their index, and the last queries of a sequence have the most keys: they go first
  int idx = gridDim.x - 1 - blockIdx.x, seq = -1, q0 = 0, nq = 0;
  for (int s = 0; s < a.n_seqs; ++s) {
    const int b = a.cu_seqlens[s], e = a.cu_seqlens[s + 1], nt = (e - b + 63) >> 6;
    if (idx < nt) {
      seq = s;
      q0 = b + idx * 64;
      nq = min(64, e - q0);
      break;
    }
    idx -= nt;
  }
  if (seq < 0) return;
  const int* bt = a.block_table + (size_t)seq * a.bt_stride;
  const int p_first = a.positions[q0], p_last = p_first + nq - 1;
  const bool valid = wave * 16 + c < nq;
  const bool wave_on = wave * 16 < nq;
  const int tq = valid ? q0 + wave * 16 + c : q0;
  const int qpos = a.positions[tq];
  const int keepf = (a.window > 0 && a.chunk == 0) ? a.keep_first : 0;
  const int lo_q = a.chunk > 0 ? (qpos / a.chunk) * a.chunk : (a.window > 0 ? qpos + 1 - a.window : 0);
  float slope[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) slope[hh] = a.slopes ? a.slopes[h0 + hh] : 0.f;

  // the key blocks: the first n_first of the kept positions, then t_lo .. t_hi
  const int lo = a.chunk > 0 ? (p_first / a.chunk) * a.chunk : (a.window > 0 ? max(0, p_first + 1 - a.window) : 0);
  const int nf = keepf > 0 ? min(keepf, lo) : 0;
  const int t_lo = lo / KT, t_hi = p_last / KT;
  const int n_first = min(nf > 0 ? (nf - 1) / KT + 1 : 0, t_lo);
  const int n_steps = n_first + t_hi - t_lo + 1;

  // the wave's queries as the second operand of S^T = K Q^T: column c, dimensions ks*32 + g*8 .. +7
  u32x4 qf[HPW][KS];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int dim = ks * 32 + g * 8;
      qf[hh][ks] = u32x4{0u, 0u, 0u, 0u};
      if (dim < D) qf[hh][ks] = *reinterpret_cast<const u32x4*>(a.q + ((size_t)tq * a.nH + h0 + hh) * D + dim);
    }
  }

  // the row of position kp in the pools, in rows of one kv head's page (a shift and a mask for the usual page sizes)
  auto row_of = [&](int kp, int head) -> size_t {
    const int pi = a.page_shift >= 0 ? kp >> a.page_shift : kp / a.page_size;
    const int sl = a.page_shift >= 0 ? kp & (a.page_size - 1) : kp % a.page_size;
    return ((size_t)bt[pi] * a.nKV + head) * a.page_size + sl;
  };
  // With pages of a power of two of at least 32 positions a step's 32 keys lie in one page: its number is looked up
  // a step ahead of the loads that need it (one dependent load less in a step's way).
  const bool one_page = a.page_shift >= 5;
  auto page_of_step = [&](int step) -> int {
    const int key0 = (step < n_first ? step : t_lo + step - n_first) * KT;
    return (one_page && step < n_steps) ? bt[key0 >> a.page_shift] : 0;
  };
  u32x4 pk[NKC], pv[NVC];
  auto fetch = [&](int step, int page) {
    const int key0 = (step < n_first ? step : t_lo + step - n_first) * KT;
#pragma unroll
    for (int n = 0; n < NKC; ++n) {
      const int id = tid + n * 256, key = id / (DP / 8), dim = (id % (DP / 8)) * 8, kp = key0 + key;
      pk[n] = u32x4{0u, 0u, 0u, 0u};
      if (dim < D && kp <= p_last) {
        const size_t row = one_page ? ((size_t)page * a.nKV + kvh) * a.page_size + (kp & (a.page_size - 1)) : row_of(kp, kvh);
        pk[n] = *reinterpret_cast<const u32x4*>(a.k_pool + row * D + dim);
      }
    }
#pragma unroll
    for (int n = 0; n < NVC; ++n) {
      const int id = tid + n * 256, key = id % KT, e = (id / KT) * 8, kp = key0 + key;     // neighbouring lanes: neighbouring keys
      pv[n] = u32x4{0u, 0u, 0u, 0u};
      if (e < DV && kp <= p_last) {
        const size_t row = one_page ? ((size_t)page * a.nKV + vh) * a.page_size + (kp & (a.page_size - 1)) : row_of(kp, vh);
        pv[n] = *reinterpret_cast<const u32x4*>(a.v_pool + row * DV + e);
      }
    }
  };

  f32x4 oT[HPW][ET];
  float m_run[HPW], l_run[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    m_run[hh] = -INFINITY;
    l_run[hh] = 0.f;
#pragma unroll
    for (int et = 0; et < ET; ++et) oT[hh][et] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  auto stage = [&](int buf) {                           // what was fetched goes into LDS
#pragma unroll
    for (int n = 0; n < NKC; ++n) {
      const int id = tid + n * 256, key = id / (DP / 8), dim = (id % (DP / 8)) * 8;
      *reinterpret_cast<u32x4*>(&Ks[buf][key][dim]) = pk[n];
    }
#pragma unroll
    for (int n = 0; n < NVC; ++n) {
      const int id = tid + n * 256, key = id % KT, e = (id / KT) * 8;
      const int col = ((key & 15) >> 2) * 8 + (key & 3) + 4 * (key >> 4);       // the order of the score tiles' rows
      const uint32_t w[4] = {pv[n][0], pv[n][1], pv[n][2], pv[n][3]};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        Vt[buf][e + 2 * i][col].bits = (uint16_t)(w[i] & 0xffffu);
        Vt[buf][e + 2 * i + 1][col].bits = (uint16_t)(w[i] >> 16);
      }
    }
  };

  fetch(0, page_of_step(0));
  int page_next = page_of_step(1);
  stage(0);
  __syncthreads();
  for (int step = 0; step < n_steps; ++step) {
    const int key0 = (step < n_first ? step : t_lo + step - n_first) * KT;
    const int cur = NBUF == 2 ? (step & 1) : 0;
    const bool more = step + 1 < n_steps;
    if (more) fetch(step + 1, page_next);
    page_next = page_of_step(step + 2);
    if (wave_on) {
      f32x4 sT[HPW][2];
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) sT[hh][0] = sT[hh][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const u32x4 kf = *reinterpret_cast<const u32x4*>(&Ks[cur][mt * 16 + c][ks * 32 + g * 8]);
#pragma unroll
          for (int hh = 0; hh < HPW; ++hh) sT[hh][mt] = mfma32(kf, qf[hh][ks], sT[hh][mt]);
        }
      }
      // which of the lane's eight keys its query sees (the same for every head)
      bool vis[8];
      bool any = false;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int kp = key0 + (j >> 2) * 16 + g * 4 + (j & 3);
        vis[j] = valid && kp <= qpos && (kp >= lo_q || kp < keepf);
        any = any || vis[j];
      }
      if (__ballot(any) != 0ull) {                       // else none of the wave's queries sees a key of this block
        u32x4 pf[HPW];
        float corr[HPW];
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
          float sc[8], m_t = -INFINITY;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            float sv = sT[hh][j >> 2][j & 3] * a.scale;
            if (a.slopes) sv = fmaf(slope[hh], (float)(key0 + (j >> 2) * 16 + g * 4 + (j & 3) - qpos), sv);
            sc[j] = vis[j] ? sv : -INFINITY;
            m_t = fmaxf(m_t, sc[j]);
          }
          m_t = fmaxf(m_t, __shfl_xor(m_t, 16, 64));
          m_t = fmaxf(m_t, __shfl_xor(m_t, 32, 64));
          const float m_new = fmaxf(m_run[hh], m_t);
          float sum = 0.f;
          uint32_t pw[4] = {0u, 0u, 0u, 0u};
          corr[hh] = 1.f;
          if (m_new > -INFINITY) {
            corr[hh] = __expf(m_run[hh] - m_new);       // m_run = -inf gives 0
            float p[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              p[j] = __expf(sc[j] - m_new);
              sum += p[j];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) pw[j] = pack_bf16x2(p[2 * j], p[2 * j + 1]);
            m_run[hh] = m_new;
          }
          l_run[hh] = fmaf(l_run[hh], corr[hh], sum);
          pf[hh] = u32x4{pw[0], pw[1], pw[2], pw[3]};
        }
#pragma unroll
        for (int et = 0; et < ET; ++et) {
          const u32x4 vf = *reinterpret_cast<const u32x4*>(&Vt[cur][et * 16 + c][g * 8]);
#pragma unroll
          for (int hh = 0; hh < HPW; ++hh) {
#pragma unroll
            for (int i = 0; i < 4; ++i) oT[hh][et][i] *= corr[hh];
            oT[hh][et] = mfma32(vf, pf[hh], oT[hh][et]);
          }
        }
      }
    }
    if (NBUF == 1) __syncthreads();                     // one buffer: everybody has read it before it is filled again
    if (more) stage(NBUF == 2 ? (cur ^ 1) : 0);
    __syncthreads();
  }

  if (!valid) return;
  const size_t t = (size_t)tq;
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    const int h = h0 + hh;
    float l_tot = l_run[hh];
    l_tot += __shfl_xor(l_tot, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    float factor = 1.f;
    if (a.sink) {                                       // one more term of the denominator, without a value
      const float sk = a.sink[h];
      const float m_fin = fmaxf(m_run[hh], sk);
      factor = __expf(m_run[hh] - m_fin);
      l_tot = fmaf(l_tot, factor, __expf(sk - m_fin));
    }
    const float inv = l_tot > 0.f ? factor / l_tot : 0.f;
#pragma unroll
    for (int et = 0; et < ET; ++et) {
      const int e = et * 16 + g * 4;
      if (e >= DV) continue;
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = oT[hh][et][i] * inv;
      if (a.vcos) {                                     // the pairs (e, e + 1) turned back by the query's position
#pragma unroll
        for (int i = 0; i < 4; i += 2) {
          const float cs = a.vcos[(size_t)qpos * (DV >> 1) + ((e + i) >> 1)], sn = a.vsin[(size_t)qpos * (DV >> 1) + ((e + i) >> 1)];
          const float u = o[i], v = o[i + 1];
          o[i] = fmaf(u, cs, __fmul_rn(v, sn));
          o[i + 1] = fmaf(v, cs, -__fmul_rn(u, sn));
        }
      }
      if (a.out32) {
        *reinterpret_cast<f32x4*>(a.out32 + ((t * a.nH + h) * a.nKV + vh) * DV + e) = f32x4{o[0], o[1], o[2], o[3]};
        continue;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (a.gate) o[i] *= sigmoid_f(a.gate[t * a.gate_stride + (a.gate_mode == 2 ? h * DV + e + i : h)], false);
        o[i] *= a.out_scale;
      }
      uint2 pkd = {pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
      *reinterpret_cast<uint2*>(a.out + (t * a.nH + h) * DV + e) = pkd;
    }
  }
}

int pad_size(int n) { return n <= 64 ? 64 : (n <= 128 ? 128 : 256); }

}  // namespace

extern "C" int alice_attention_tiled_supported(int d, int dv) {
  return d >= 8 && dv >= 8 && d % 8 == 0 && dv % 8 == 0 && d <= 256 && dv <= 256;
}

// q: bfloat16 [T, nH d]; pools: bfloat16 [pages, nKV, page, d / dv] row-major; out: bfloat16 [T, nH dv], or out32:
// float32 [T, nH, nKV, dv] (then nothing goes to out and no gate is applied); gate: float32 rows.  The step's tokens
// are those of n_seqs sequences in order (cu_seqlens), each at consecutive positions.  heads_per_wave: 0 is the
// launcher's choice (1); 2 or 4 ask for that many heads of a group a wave.
extern "C" int alice_attention_tiled(const void* q, const void* k_pool, const void* v_pool, void* out, float* out32,
                                     const int* positions, const int* cu_seqlens, const int* block_table, int bt_stride,
                                     int T, int n_seqs, int nH, int nKV, int d, int dv, int page_size, float scale, int window,
                                     int chunk, int keep_first, const float* bias_slopes, const float* sink,
                                     const float* vrot_cos, const float* vrot_sin, const float* gate, int gate_stride,
                                     int gate_mode, float out_scale, int heads_per_wave, hipStream_t stream) {
  ALICE_CHECK(alice_attention_tiled_supported(d, dv), "attention: head sizes %d and %d are outside this kernel's range (multiples of 8 up to 256)", d, dv);
  ALICE_CHECK(q && k_pool && v_pool && (out || out32) && positions && cu_seqlens && block_table, "attention: a pointer is missing");
  ALICE_CHECK(T >= 0 && n_seqs >= 1 && nH >= 1 && nKV >= 1 && nH % nKV == 0, "attention: bad head counts nH=%d nKV=%d", nH, nKV);
  ALICE_CHECK(nH <= 65535 && nKV <= 65535, "attention: too many heads for one launch (%d)", nH);
  ALICE_CHECK(page_size > 0 && bt_stride > 0, "attention: bad page geometry");
  ALICE_CHECK(window >= 0 && chunk >= 0 && keep_first >= 0, "attention: window, chunk and keep_first must not be negative (0 turns them off)");
  ALICE_CHECK((vrot_cos == nullptr) == (vrot_sin == nullptr), "attention: turning the output back needs both tables");
  ALICE_CHECK(gate == nullptr || (gate_mode == 1 && gate_stride >= nH) || (gate_mode == 2 && gate_stride >= nH * dv),
              "attention: gate rows of %d elements are too short", gate_stride);
  ALICE_CHECK(((uintptr_t)q & 15) == 0 && ((uintptr_t)k_pool & 15) == 0 && ((uintptr_t)v_pool & 15) == 0 &&
              ((uintptr_t)out & 7) == 0 && ((uintptr_t)out32 & 15) == 0, "attention: operands are not aligned");
  if (T == 0) return 0;
  int page_shift = -1;
  for (int b = 0; b < 31; ++b)
    if (page_size == (1 << b)) page_shift = b;
  TiledArgs a{(const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, (bf16_t*)out, out32, positions, cu_seqlens,
              block_table, bt_stride, n_seqs, nH, nKV, d, dv, page_size, scale, window, chunk, keep_first, page_shift, bias_slopes, sink,
              vrot_cos, vrot_sin, gate, gate_stride, gate_mode, out_scale};
  const int dp = pad_size(d), dvp = pad_size(dv);
  // Heads of a kv head's group a wave: one.  Two or four (each staged key block and every fragment read of it then
  // serves them all) measured slower at head sizes of 128, for want of registers (one wave a SIMD instead of three):
  // one prompt of 2,048 tokens 86 us with one head a wave, 108 with two; eight prompts 552 against 744 with four.
  const int per = nH / nKV;
  int hpw = 1;
  if (heads_per_wave > 0) {                             // the caller's choice (tests)
    ALICE_CHECK((heads_per_wave == 1 || heads_per_wave == 2 || heads_per_wave == 4) && per % heads_per_wave == 0 &&
                (heads_per_wave == 1 || (dp <= 128 && dvp <= 128)),
                "attention: %d heads a wave do not divide the group of %d, or the head sizes are beyond 128", heads_per_wave, per);
    hpw = heads_per_wave;
  }
  dim3 grid(ceil_div(T, 64) + n_seqs, nH / hpw, out32 ? nKV : 1);
#define GO(DP, DVP)                                                         \
  do {                                                                      \
    if constexpr (DP <= 128 && DVP <= 128) {                                \
      if (hpw == 4) attn_tiled_kernel<DP, DVP, 4><<<grid, 256, 0, stream>>>(a);      \
      else if (hpw == 2) attn_tiled_kernel<DP, DVP, 2><<<grid, 256, 0, stream>>>(a); \
      else attn_tiled_kernel<DP, DVP, 1><<<grid, 256, 0, stream>>>(a);               \
    } else {                                                                \
      attn_tiled_kernel<DP, DVP, 1><<<grid, 256, 0, stream>>>(a);           \
    }                                                                       \
  } while (0)
#define BY_DV(DP)                     \
  do {                                \
    if (dvp == 64) GO(DP, 64);        \
    else if (dvp == 128) GO(DP, 128); \
    else GO(DP, 256);                 \
  } while (0)
  if (dp == 64) BY_DV(64);
  else if (dp == 128) BY_DV(128);
  else BY_DV(256);
#undef BY_DV
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}
