// N-dimensional axis permutation on the device: dst[i_perm[0], ..., i_perm[n-1]]
// = src[i_0, ..., i_{n-1}].  The Function classes use it for the tensor
// layouts the normalization kernels do not read in place (the reference brings
// those to channel-first through the core's ChannelFirstAdaptor,
// src/nbla/cuda/function/generic/group_normalization.cu:40-55,93-109, whose
// device work is the generic transpose of
// include/nbla/cuda/function/kernel/transpose.cuh:19-53).
//
// Two kernels.  When source and destination share their innermost axis, every
// thread copies elements of one run along it (both sides coalesced).  When
// they differ, a block moves a 64 x 64 tile spanned by the two innermost axes
// through LDS: read along the source's innermost axis, written along the
// destination's, so both sides see whole cache lines; the reference's kernel
// gathers element by element with one side strided.
#include <algorithm>

#include "common.cuh"
#include "launch.hpp"

namespace nblahip {
namespace {

constexpr int kMaxPermuteDims = 8;

struct PermuteOuter {
  // Axes other than the two tile axes (or, for the run kernel, all axes of the
  // destination but the innermost), outermost first: extent as a divider and
  // element strides on both sides.
  FastDiv dim[kMaxPermuteDims];
  uint32_t src_stride[kMaxPermuteDims];
  uint32_t dst_stride[kMaxPermuteDims];
  int n;
};

template <typename T> __device__ __forceinline__ T add_elem(T a, T b) {
  return from_f32<T>(to_f32<T>(a) + to_f32<T>(b));
}

// Same innermost axis on both sides: the destination is walked linearly,
// `inner` consecutive elements at a time mapping to consecutive source
// elements.
template <typename T, bool ACCUM>
__global__ void __launch_bounds__(256)
permute_run_kernel(const T *__restrict__ src, T *__restrict__ dst, uint32_t total, FastDiv inner,
                   const PermuteOuter o) {
  for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < total; i += gridDim.x * 256u) {
    uint32_t r = inner.div(i);
    uint32_t s = i - r * inner.d;
#pragma unroll 1
    for (int k = o.n - 1; k >= 0; --k) {
      const uint32_t q = o.dim[k].div(r);
      s += (r - q * o.dim[k].d) * o.src_stride[k];
      r = q;
    }
    const T v = src[s];
    dst[i] = ACCUM ? add_elem<T>(dst[i], v) : v;
  }
}

// Different innermost axes.  Axis A is the source's innermost one (extent na,
// destination stride dst_a), axis B the destination's (extent nb, source
// stride src_b).  blockIdx.x enumerates (outer index, tile of B, tile of A),
// the tile of A fastest.
template <typename T, bool ACCUM>
__global__ void __launch_bounds__(256)
permute_tile_kernel(const T *__restrict__ src, T *__restrict__ dst, uint32_t na, uint32_t nb,
                    uint32_t src_b, uint32_t dst_a, FastDiv tiles_a, FastDiv tiles_b,
                    const PermuteOuter o) {
  __shared__ T tile[64][65];
  uint32_t r = tiles_a.div(blockIdx.x);
  const uint32_t a0 = (blockIdx.x - r * tiles_a.d) * 64u;
  const uint32_t q = tiles_b.div(r);
  const uint32_t b0 = (r - q * tiles_b.d) * 64u;
  r = q;
  size_t sbase = 0, dbase = 0;
#pragma unroll 1
  for (int k = o.n - 1; k >= 0; --k) {
    const uint32_t qq = o.dim[k].div(r);
    const uint32_t idx = r - qq * o.dim[k].d;
    sbase += static_cast<size_t>(idx) * o.src_stride[k];
    dbase += static_cast<size_t>(idx) * o.dst_stride[k];
    r = qq;
  }
  const uint32_t tx = threadIdx.x & 63u, ty = threadIdx.x >> 6;
#pragma unroll 4
  for (uint32_t j = ty; j < 64u; j += 4u) {
    const uint32_t a = a0 + tx, b = b0 + j;
    if (a < na && b < nb) tile[j][tx] = src[sbase + static_cast<size_t>(b) * src_b + a];
  }
  __syncthreads();
#pragma unroll 4
  for (uint32_t j = ty; j < 64u; j += 4u) {
    const uint32_t a = a0 + j, b = b0 + tx;
    if (a < na && b < nb) {
      T *p = dst + dbase + static_cast<size_t>(a) * dst_a + b;
      const T v = tile[tx][j];
      *p = ACCUM ? add_elem<T>(*p, v) : v;
    }
  }
}

template <typename T>
int permute_t(const void *src_v, void *dst_v, int nd, const int64_t *dims, const int64_t *sstr,
              int accum, hipStream_t st) {
  // dims / sstr: the destination's axes, outermost first, with the source
  // stride of each (already merged where possible); nd >= 1.
  const T *src = static_cast<const T *>(src_v);
  T *dst = static_cast<T *>(dst_v);
  int64_t total = 1;
  int64_t dstr[kMaxPermuteDims];
  for (int i = nd - 1; i >= 0; --i) {
    dstr[i] = total;
    total *= dims[i];
  }
  PermuteOuter o{};
  if (sstr[nd - 1] == 1) {
    for (int i = 0; i < nd - 1; ++i) {
      o.dim[i] = FastDiv(static_cast<uint32_t>(dims[i]));
      o.src_stride[i] = static_cast<uint32_t>(sstr[i]);
      o.dst_stride[i] = static_cast<uint32_t>(dstr[i]);
    }
    o.n = nd - 1;
    const int64_t blocks = std::min<int64_t>((total + 255) / 256, int64_t{device_cus()} * 32);
    if (accum) {
      NBLAHIP_LAUNCH("permute_run_kernel", (permute_run_kernel<T, true>),
                     dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, src, dst,
                     static_cast<uint32_t>(total), FastDiv(static_cast<uint32_t>(dims[nd - 1])), o);
    } else {
      NBLAHIP_LAUNCH("permute_run_kernel", (permute_run_kernel<T, false>),
                     dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, src, dst,
                     static_cast<uint32_t>(total), FastDiv(static_cast<uint32_t>(dims[nd - 1])), o);
    }
    return last_launch_status();
  }
  // The source's innermost axis sits at position pa of the destination.
  int pa = -1;
  for (int i = 0; i < nd - 1; ++i)
    if (sstr[i] == 1) pa = i;
  if (pa < 0) return NBLAHIP_EINVAL;
  const uint32_t na = static_cast<uint32_t>(dims[pa]), nb = static_cast<uint32_t>(dims[nd - 1]);
  int n = 0;
  int64_t outer = 1;
  for (int i = 0; i < nd - 1; ++i) {
    if (i == pa) continue;
    o.dim[n] = FastDiv(static_cast<uint32_t>(dims[i]));
    o.src_stride[n] = static_cast<uint32_t>(sstr[i]);
    o.dst_stride[n] = static_cast<uint32_t>(dstr[i]);
    outer *= dims[i];
    ++n;
  }
  o.n = n;
  const uint32_t ta = (na + 63) / 64, tb = (nb + 63) / 64;
  const int64_t blocks = outer * ta * tb;
  if (blocks >= (int64_t{1} << 31)) return NBLAHIP_ERANGE;
  if (accum) {
    NBLAHIP_LAUNCH("permute_tile_kernel", (permute_tile_kernel<T, true>),
                   dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, src, dst, na, nb,
                   static_cast<uint32_t>(sstr[nd - 1]), static_cast<uint32_t>(dstr[pa]), FastDiv(ta),
                   FastDiv(tb), o);
  } else {
    NBLAHIP_LAUNCH("permute_tile_kernel", (permute_tile_kernel<T, false>),
                   dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, src, dst, na, nb,
                   static_cast<uint32_t>(sstr[nd - 1]), static_cast<uint32_t>(dstr[pa]), FastDiv(ta),
                   FastDiv(tb), o);
  }
  return last_launch_status();
}

} // namespace
} // namespace nblahip

using namespace nblahip;

extern "C" int nblahip_permute(const void *src, void *dst, int ndim, const int64_t *shape,
                               const int *perm, int accum, int dtype, void *stream) {
  if (dtype != NBLAHIP_F32 && dtype != NBLAHIP_F16) return NBLAHIP_EINVAL;
  if (ndim < 1 || ndim > kMaxPermuteDims || !shape || !perm) return NBLAHIP_EINVAL;
  bool seen[kMaxPermuteDims] = {false};
  __int128 total = 1;
  for (int i = 0; i < ndim; ++i) {
    if (perm[i] < 0 || perm[i] >= ndim || seen[perm[i]] || shape[i] < 0) return NBLAHIP_EINVAL;
    seen[perm[i]] = true;
    total *= shape[i];
  }
  if (total == 0) return 0;
  if (total > (static_cast<__int128>(1) << 31) - 1) return NBLAHIP_ERANGE;
  if (!src || !dst) return NBLAHIP_EINVAL;
  if (src == dst) return NBLAHIP_EALIAS;
  // Source strides, then the destination's axes with their source strides;
  // axes of extent 1 dropped, neighbours that stay neighbours merged.
  int64_t sstride[kMaxPermuteDims];
  int64_t run = 1;
  for (int i = ndim - 1; i >= 0; --i) {
    sstride[i] = run;
    run *= shape[i];
  }
  int64_t dims[kMaxPermuteDims], sstr[kMaxPermuteDims];
  int nd = 0;
  for (int i = 0; i < ndim; ++i) {
    const int ax = perm[i];
    if (shape[ax] == 1) continue;
    if (nd > 0 && sstr[nd - 1] == sstride[ax] * shape[ax]) {
      dims[nd - 1] *= shape[ax];
      sstr[nd - 1] = sstride[ax];
    } else {
      dims[nd] = shape[ax];
      sstr[nd] = sstride[ax];
      ++nd;
    }
  }
  if (nd == 0) { // a single element
    dims[0] = 1;
    sstr[0] = 1;
    nd = 1;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return dtype == NBLAHIP_F16 ? permute_t<__half>(src, dst, nd, dims, sstr, accum, st)
                              : permute_t<float>(src, dst, nd, dims, sstr, accum, st);
}
