// From the padding-free token stream back to the [batch, response_length] window.
//
// With remove-padding the head returns one value per attended token, in the order of `indices`
// (the flat positions b * seqlen + s of the attended tokens, ascending, as unpad_input produces
// them).  The actor then rebuilds a [batch, seqlen] tensor with pad_input and keeps the columns
// [-response_length - 1, -1) (verl/workers/actor/dp_actor.py:316-344).  Here each output element
// looks its flat position up in `indices` by binary search and takes the token's value or 0, so
// the window is written once, with coalesced stores and no zero-fill pass, for up to three
// per-token tensors (log-prob, entropy, sum of squared probabilities) in one launch.  The backward
// direction is a plain gather: d_token[i] = d_window[b][j] if token i lies in the window.
#include "common.h"

namespace vamd {

struct Window {
  const int64_t* indices;  // [nnz] ascending flat positions
  int64_t nnz, batch, seqlen, width;
};

__global__ __launch_bounds__(256) void window_scatter_kernel(Window w, const float* __restrict__ a,
                                                             const float* __restrict__ b,
                                                             const float* __restrict__ c, float* __restrict__ oa,
                                                             float* __restrict__ ob, float* __restrict__ oc) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= w.batch * w.width) return;
  const int64_t row = e / w.width, j = e % w.width;
  const int64_t col = w.seqlen - w.width - 1 + j;
  float va = 0.f, vb = 0.f, vc = 0.f;
  if (col >= 0) {
    const int64_t want = row * w.seqlen + col;
    int64_t lo = 0, hi = w.nnz;  // first position with indices[pos] >= want
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (w.indices[mid] < want) lo = mid + 1; else hi = mid;
    }
    if (lo < w.nnz && w.indices[lo] == want) {
      va = a[lo];
      if (b) vb = b[lo];
      if (c) vc = c[lo];
    }
  }
  oa[e] = va;
  if (ob) ob[e] = vb;
  if (oc) oc[e] = vc;
}

__global__ __launch_bounds__(256) void window_gather_kernel(Window w, const float* __restrict__ da,
                                                            const float* __restrict__ db, float* __restrict__ ta,
                                                            float* __restrict__ tb) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= w.nnz) return;
  const int64_t p = w.indices[i];
  const int64_t row = p / w.seqlen, col = p % w.seqlen;
  const int64_t j = col - (w.seqlen - w.width - 1);
  const bool in = j >= 0 && j < w.width && row >= 0 && row < w.batch;
  if (ta) ta[i] = in ? da[row * w.width + j] : 0.f;
  if (tb) tb[i] = in ? db[row * w.width + j] : 0.f;
}

}  // namespace vamd

using namespace vamd;

static int check_window(const char* what, const int64_t* indices, int64_t nnz, int64_t batch, int64_t seqlen,
                        int64_t width) {
  VAMD_REQUIRE(indices && nnz >= 0 && batch > 0 && seqlen > 0, "%s: bad argument", what);
  VAMD_REQUIRE(width > 0 && width <= seqlen, "%s: response_length %lld does not fit seqlen %lld", what,
               (long long)width, (long long)seqlen);
  VAMD_REQUIRE(nnz <= batch * seqlen, "%s: more tokens than positions", what);
  return VAMD_OK;
}

extern "C" int vamd_response_window_scatter(const float* a, const float* b, const float* c, const int64_t* indices,
                                            int64_t nnz, int64_t batch, int64_t seqlen, int64_t response_length,
                                            float* out_a, float* out_b, float* out_c, void* stream) {
  int st = check_window("response_window_scatter", indices, nnz, batch, seqlen, response_length);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE(a && out_a && (!b == !out_b) && (!c == !out_c), "response_window_scatter: input / output mismatch");
  const Window w{indices, nnz, batch, seqlen, response_length};
  const int64_t n = batch * response_length;
  hipLaunchKernelGGL(window_scatter_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), w, a, b, c, out_a, out_b, out_c);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}

extern "C" int vamd_response_window_gather(const float* d_out_a, const float* d_out_b, const int64_t* indices,
                                           int64_t nnz, int64_t batch, int64_t seqlen, int64_t response_length,
                                           float* d_a, float* d_b, void* stream) {
  int st = check_window("response_window_gather", indices, nnz, batch, seqlen, response_length);
  if (st != VAMD_OK) return st;
  VAMD_REQUIRE((!d_a == !d_out_a) && (!d_b == !d_out_b) && (d_a || d_b), "response_window_gather: input / output mismatch");
  if (nnz == 0) return VAMD_OK;
  const Window w{indices, nnz, batch, seqlen, response_length};
  hipLaunchKernelGGL(window_gather_kernel, dim3((unsigned)((nnz + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), w, d_out_a, d_out_b, d_a, d_b);
  VAMD_LAUNCH_CHECK();
  return VAMD_OK;
}
