// (b2) fp32 reduction of the per-rank partial slices of a GEMM-RS.
//   out[e] = round(sum_i float(c[((i + first) % R) * stride + e])), i = 0..R-1, in that order.
// Follows kernel_consumer_reduce (kernels/amd/gemm_reduce_scatter.py:232-258) for the slice order
// (cur_rank = (i + rank + 1) % num_ranks) but accumulates in fp32 instead of the output dtype.
//
// HBM-bound: (R+1) * n_elems * 2 bytes per launch. Each lane owns 8 consecutive elements (one
// 16-byte vector) of two positions a workgroup-stride apart and keeps all R*2 loads in flight
// before the first add, so a wave has 2*R KiB outstanding.
#include "common.h"

namespace tdist {

constexpr int kReduceThreads = 256;
constexpr int kReduceUnroll = 2;
#ifndef TDIST_REDUCE_RESIDENT
#define TDIST_REDUCE_RESIDENT 6
#endif
constexpr int kReduceResident = TDIST_REDUCE_RESIDENT;

template <typename T>
__device__ __forceinline__ void accumulate8(float* acc, const int4v& v) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t w = (uint32_t)v[j];
    acc[2 * j] += T::lo(w);
    acc[2 * j + 1] += T::hi(w);
  }
}

template <typename T, int R>
__global__ __launch_bounds__(kReduceThreads) void reduce_slices_fixed_kernel(const int4v* __restrict__ c,
                                                                              int64_t stride16, int first,
                                                                              int64_t n16, int4v* __restrict__ out) {
  for (int64_t blk = blockIdx.x; blk * (kReduceThreads * kReduceUnroll) < n16; blk += gridDim.x) {
  const int64_t base = blk * (kReduceThreads * kReduceUnroll) + threadIdx.x;
  int4v v[kReduceUnroll][R];
#pragma unroll
  for (int u = 0; u < kReduceUnroll; ++u) {
    const int64_t e = base + u * kReduceThreads;
    if (e < n16) {
      int s = first;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        v[u][i] = __builtin_nontemporal_load(c + (int64_t)s * stride16 + e);
        s = (s + 1 == R) ? 0 : s + 1;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < kReduceUnroll; ++u) {
    const int64_t e = base + u * kReduceThreads;
    if (e < n16) {
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < R; ++i) accumulate8<T>(acc, v[u][i]);
      int4v o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = (int)T::pack(acc[2 * j], acc[2 * j + 1]);
      __builtin_nontemporal_store(o, out + e);
    }
  }
  }
}

// Any slice count, any element count, any alignment: one element per thread.
template <typename T>
__global__ __launch_bounds__(kReduceThreads) void reduce_slices_generic_kernel(const unsigned short* __restrict__ c,
                                                                                int64_t stride, int n_slices,
                                                                                int first, int64_t n_elems,
                                                                                unsigned short* __restrict__ out) {
  const int64_t e = (int64_t)blockIdx.x * kReduceThreads + threadIdx.x;
  if (e >= n_elems) return;
  float acc = 0.f;
  int s = first;
  for (int i = 0; i < n_slices; ++i) {
    acc += T::one(c[(int64_t)s * stride + e]);
    s = (s + 1 == n_slices) ? 0 : s + 1;
  }
  out[e] = (unsigned short)(T::pack(acc, 0.f) & 0xffffu);
}

template <typename T>
static int launch_reduce(const void* c, int64_t slice_stride, int n_slices, int first_slice, int64_t n_elems,
                         void* out, hipStream_t stream) {
  const bool vec_ok = aligned16(c) && aligned16(out) && (slice_stride % 8 == 0) && (n_elems % 8 == 0);
  const int64_t n16 = n_elems / 8;
  const int64_t per_block = kReduceThreads * kReduceUnroll;
  const int64_t blocks = ceil_div(n16, per_block);
  // at most six workgroups per compute unit (what the kernel's registers allow to be resident), each looping over
  // its share, so that the last round is not a third-full one
  const DeviceInfo& di = device_info();
  const int64_t resident = (int64_t)(di.ok == 1 ? di.num_cus : 256) * kReduceResident;
  const int64_t grid = blocks < resident ? blocks : resident;
  if (vec_ok && blocks <= 0x7fffffff) {
#define TDIST_REDUCE_CASE(R)                                                                                   \
  case R:                                                                                                      \
    hipLaunchKernelGGL((reduce_slices_fixed_kernel<T, R>), dim3((unsigned)grid), dim3(kReduceThreads), 0,      \
                       stream, (const int4v*)c, slice_stride / 8, first_slice, n16, (int4v*)out);              \
    return launch_status("tdist_reduce_slices");
    switch (n_slices) {
      TDIST_REDUCE_CASE(1)
      TDIST_REDUCE_CASE(2)
      TDIST_REDUCE_CASE(4)
      TDIST_REDUCE_CASE(8)
      TDIST_REDUCE_CASE(16)
      default:
        break;
    }
#undef TDIST_REDUCE_CASE
  }
  const int64_t gblocks = ceil_div(n_elems, kReduceThreads);
  if (gblocks > 0x7fffffff) return fail(TDIST_ERR_UNSUPPORTED, "tdist_reduce_slices: too many elements");
  hipLaunchKernelGGL((reduce_slices_generic_kernel<T>), dim3((unsigned)gblocks), dim3(kReduceThreads), 0, stream,
                     (const unsigned short*)c, slice_stride, n_slices, first_slice, n_elems, (unsigned short*)out);
  return launch_status("tdist_reduce_slices(generic)");
}

}  // namespace tdist

using namespace tdist;

extern "C" int tdist_reduce_slices(const void* c, int64_t slice_stride, int n_slices, int first_slice,
                                   int64_t n_elems, void* out, int dtype, void* stream) {
  if (!c || !out) return fail(TDIST_ERR_INVALID, "tdist_reduce_slices: null pointer");
  if (n_slices <= 0 || n_elems < 0 || slice_stride < 0)
    return fail(TDIST_ERR_INVALID, "tdist_reduce_slices: n_slices must be > 0, sizes >= 0");
  if (first_slice < 0 || first_slice >= n_slices)
    return fail(TDIST_ERR_INVALID, "tdist_reduce_slices: first_slice %d outside [0,%d)", first_slice, n_slices);
  if (n_elems == 0) return TDIST_OK;
  if (dtype == TDIST_BF16) return launch_reduce<BF16>(c, slice_stride, n_slices, first_slice, n_elems, out, (hipStream_t)stream);
  if (dtype == TDIST_F16) return launch_reduce<F16>(c, slice_stride, n_slices, first_slice, n_elems, out, (hipStream_t)stream);
  return fail(TDIST_ERR_UNSUPPORTED, "tdist_reduce_slices: dtype %d (bf16 and f16 only)", dtype);
}
