// Several branches added to the residual stream at once: x += sum_j norm_j(b_j), each branch the sum of its
// partial results and, where it has a weight, RMS-normed over the row first:
//   norm_j(b) = b / sqrt(mean(b^2) + eps_j) * (off_j + w_j).
// The layer arrangement whose mixer and feed-forward read one norm's output side by side ends in such a sum; one
// kernel instead of one per branch.  Optionally the new x is also written out in the activation dtype (what the
// next part reads).  One block per row of up to 8192 elements, all sums 32-bit in a fixed order.
#include "common.h"
#include "alice_hip.h"

namespace {

struct Branches {
  const float* b[ALICE_MAX_BRANCHES];
  const void* w[ALICE_MAX_BRANCHES];
  long stride[ALICE_MAX_BRANCHES];
  int parts[ALICE_MAX_BRANCHES];
  float eps[ALICE_MAX_BRANCHES];
  float off[ALICE_MAX_BRANCHES];
  int n;
};

// The row in registers, EPT elements a thread (element tid + e * blockDim.x), every load of a (branch, partial
// result) issued together.
template <typename TW, typename TO, bool FULL, int EPT>
__global__ __launch_bounds__(1024) void add_branches_kernel(float* __restrict__ resid, Branches a, TO* __restrict__ out, int H) {
  __shared__ float red[17];
  const size_t row = (size_t)blockIdx.x * H;
  float v[ALICE_MAX_BRANCHES][EPT];
  float x[EPT];
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = threadIdx.x + e * blockDim.x;
    x[e] = i < H ? resid[row + i] : 0.f;
  }
#pragma unroll
  for (int j = 0; j < ALICE_MAX_BRANCHES; ++j) {
#pragma unroll
    for (int e = 0; e < EPT; ++e) v[j][e] = 0.f;
    if (j < a.n) {
      // eight partial results at a time, every load of the eight issued before the first sum
      for (int p0 = 0; p0 < a.parts[j]; p0 += 8) {
        float t[8][EPT];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const float* src = a.b[j] + (size_t)min(p0 + u, a.parts[j] - 1) * a.stride[j] + row;
#pragma unroll
          for (int e = 0; e < EPT; ++e) {
            const int i = threadIdx.x + e * blockDim.x;
            t[u][e] = (i < H && p0 + u < a.parts[j]) ? src[i] : 0.f;
          }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
          for (int e = 0; e < EPT; ++e) v[j][e] += t[u][e];
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < ALICE_MAX_BRANCHES; ++j) {
    if (j < a.n && a.w[j]) {                                   // uniform over the block
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < EPT; ++e) ss = fmaf(v[j][e], v[j][e], ss);
      const float s = block_sum(ss, red) / (float)H + a.eps[j];
      const float inv = FULL ? 1.f / sqrtf(s) : rsqrtf(s);
#pragma unroll
      for (int e = 0; e < EPT; ++e) {
        const int i = threadIdx.x + e * blockDim.x;
        if (i < H) x[e] += v[j][e] * inv * (a.off[j] + load_f32((const TW*)a.w[j], i));
      }
    } else if (j < a.n) {
#pragma unroll
      for (int e = 0; e < EPT; ++e) x[e] += v[j][e];
    }
  }
#pragma unroll
  for (int e = 0; e < EPT; ++e) {
    const int i = threadIdx.x + e * blockDim.x;
    if (i < H) {
      resid[row + i] = x[e];
      if (out) store_f32(out, row + i, x[e]);
    }
  }
}

}  // namespace

extern "C" int alice_add_branches(float* resid, int n, const float* const* branches, const int* n_partials,
                                  const long* partial_strides, const void* const* weights, int w_dtype,
                                  const float* eps, const float* offsets, void* out, int out_dtype, int T, int H,
                                  int full_precision, hipStream_t stream) {
  ALICE_CHECK(resid && T >= 0 && H > 0, "add_branches: bad sizes T=%d H=%d", T, H);
  ALICE_CHECK(n >= 1 && n <= ALICE_MAX_BRANCHES, "add_branches: %d branches (1 to %d)", n, ALICE_MAX_BRANCHES);
  ALICE_CHECK(dtype_ok(w_dtype) && dtype_ok(out_dtype), "add_branches: unknown dtype");
  Branches a;
  a.n = n;
  for (int j = 0; j < ALICE_MAX_BRANCHES; ++j) {
    a.b[j] = j < n ? branches[j] : nullptr;
    a.w[j] = j < n ? weights[j] : nullptr;
    a.stride[j] = j < n ? partial_strides[j] : 0;
    a.parts[j] = j < n ? n_partials[j] : 0;
    a.eps[j] = j < n ? eps[j] : 0.f;
    a.off[j] = j < n ? offsets[j] : 0.f;
    ALICE_CHECK(j >= n || (a.b[j] && a.parts[j] >= 1 && a.parts[j] <= 64), "add_branches: branch %d is missing or has a bad number of partial results", j);
  }
  if (T == 0) return 0;
  ALICE_CHECK(H <= 8192, "add_branches: rows of up to 8192 elements, found %d", H);
  const int ept = H <= 512 ? 1 : (H <= 1024 ? 2 : (H <= 4096 ? 4 : 8));
  const int threads = ceil_div(ceil_div(H, ept), 64) * 64;
#define GO(FULL)                                                                                               \
  do {                                                                                                         \
    if (ept == 1) add_branches_kernel<TW, TO, FULL, 1><<<T, threads, 0, stream>>>(resid, a, (TO*)out, H);      \
    else if (ept == 2) add_branches_kernel<TW, TO, FULL, 2><<<T, threads, 0, stream>>>(resid, a, (TO*)out, H); \
    else if (ept == 4) add_branches_kernel<TW, TO, FULL, 4><<<T, threads, 0, stream>>>(resid, a, (TO*)out, H); \
    else add_branches_kernel<TW, TO, FULL, 8><<<T, threads, 0, stream>>>(resid, a, (TO*)out, H);               \
  } while (0)
  DISPATCH_DTYPE(w_dtype, TW, DISPATCH_DTYPE(out_dtype, TO, {
    if (full_precision) GO(true); else GO(false);
  }));
#undef GO
  ALICE_LAUNCH_CHECK();
  return 0;
}
