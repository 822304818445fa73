// Transpose of quantized tensors (_QuantizedTranspose: itex/core/kernels/common/transpose_op.h:197-236).
// Pure data movement, HBM-bound: 2 bytes of traffic per tensor byte.
#include <algorithm>

#include "common.hpp"

namespace itexhip {
namespace {

constexpr int kMaxRank = 8;

struct TransposeArgs {
  int rank;                   // after merging
  int64_t out_dims[kMaxRank];
  int64_t in_stride[kMaxRank];  // stride in the input (in units) of output dimension i
  int64_t total;              // number of units
};

// One unit (UNIT bytes) per thread and iteration: the output is written linearly, the input address
// comes from the output coordinates.
template <typename unit_t>
__global__ __launch_bounds__(256) void transpose_kernel(const TransposeArgs a, const unit_t* __restrict__ x,
                                                        unit_t* __restrict__ y) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t o = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; o < a.total; o += stride) {
    int64_t rem = o, src = 0;
#pragma unroll
    for (int d = kMaxRank - 1; d >= 0; --d) {
      if (d >= a.rank) continue;
      const int64_t q = d == 0 ? 0 : rem / a.out_dims[d];
      src += (rem - q * a.out_dims[d]) * a.in_stride[d];
      rem = q;
    }
    y[o] = x[src];
  }
}

}  // namespace
}  // namespace itexhip

using namespace itexhip;

extern "C" int itexhip_transpose(const void* x, void* y, int elem_size, int rank, const int64_t* dims, const int32_t* perm,
                                 void* stream) {
  const char* who = "itexhip_transpose";
  ITEXHIP_REQUIRE(elem_size == 1 || elem_size == 4, "%s: element size %d (1 or 4)", who, elem_size);
  ITEXHIP_REQUIRE(rank >= 0 && rank <= kMaxRank, "%s: rank %d (at most %d)", who, rank, kMaxRank);
  ITEXHIP_REQUIRE(rank == 0 || (dims && perm), "%s: null dims or perm", who);
  bool seen[kMaxRank] = {false};
  int64_t total = 1;
  for (int i = 0; i < rank; ++i) {
    ITEXHIP_REQUIRE(perm[i] >= 0 && perm[i] < rank && !seen[perm[i]], "%s: perm is not a permutation", who);
    seen[perm[i]] = true;
    ITEXHIP_REQUIRE(dims[i] >= 0, "%s: negative dimension", who);
    total *= dims[i];
  }
  if (total == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(x && y && aligned(x, elem_size) && aligned(y, elem_size), "%s: null or misaligned buffer", who);

  // input strides (elements), then the output's view of them; dimensions of extent 1 drop out
  int64_t in_stride[kMaxRank], od[kMaxRank], os[kMaxRank];
  {
    int64_t st = 1;
    for (int i = rank - 1; i >= 0; --i) { in_stride[i] = st; st *= dims[i]; }
  }
  int n = 0;
  for (int i = 0; i < rank; ++i) {
    if (dims[perm[i]] == 1) continue;
    od[n] = dims[perm[i]];
    os[n] = in_stride[perm[i]];
    // merge with the previous output dimension when the two are also adjacent, in this order, in the input
    if (n > 0 && os[n - 1] == os[n] * od[n]) {
      od[n - 1] *= od[n];
      os[n - 1] = os[n];
    } else {
      ++n;
    }
  }
  if (n == 0) { od[0] = 1; os[0] = 1; n = 1; }  // a single element

  // the innermost run: contiguous in both tensors when its input stride is 1
  int64_t bytes_inner = os[n - 1] == 1 ? od[n - 1] * elem_size : 0;
  int unit = elem_size;
  if (bytes_inner >= 16 && bytes_inner % 16 == 0 && aligned(x, 16) && aligned(y, 16)) {
    bool ok = true;  // every other stride must keep 16-byte alignment
    for (int i = 0; i + 1 < n; ++i) ok = ok && (os[i] * elem_size) % 16 == 0;
    if (ok) unit = 16;
  } else if (elem_size == 1 && bytes_inner >= 4 && bytes_inner % 4 == 0 && aligned(x, 4) && aligned(y, 4)) {
    bool ok = true;
    for (int i = 0; i + 1 < n; ++i) ok = ok && os[i] % 4 == 0;
    if (ok) unit = 4;
  }
  const int per = unit / elem_size;  // elements per unit
  TransposeArgs a{};
  a.rank = n;
  for (int i = 0; i < n; ++i) {
    a.out_dims[i] = od[i];
    a.in_stride[i] = os[i] / (i + 1 < n ? per : 1);
  }
  if (per > 1) { a.out_dims[n - 1] = od[n - 1] / per; a.in_stride[n - 1] = 1; }
  a.total = total / per;
  const int64_t blocks = std::min<int64_t>((a.total + 255) / 256, 256 * 16);
  hipStream_t st = as_stream(stream);
  if (unit == 16) transpose_kernel<i4><<<static_cast<unsigned>(blocks), 256, 0, st>>>(a, static_cast<const i4*>(x), static_cast<i4*>(y));
  else if (unit == 4) transpose_kernel<uint32_t><<<static_cast<unsigned>(blocks), 256, 0, st>>>(a, static_cast<const uint32_t*>(x), static_cast<uint32_t*>(y));
  else transpose_kernel<uint8_t><<<static_cast<unsigned>(blocks), 256, 0, st>>>(a, static_cast<const uint8_t*>(x), static_cast<uint8_t*>(y));
  ITEXHIP_CHECK_LAUNCH(who);
  return ITEXHIP_OK;
}
