// Measurement aids of the BTP library, kept apart from the operator: a plain copy kernel (hardware-counter
// calibration) and bandwidth probes that move the operator's traffic in the operator's access shape with no
// arithmetic. bench.py runs them beside the kernels to show where those stand against what the memory system
// gives; nothing in the operator calls them. Declared in include/spear_btp_probe.h. No counterpart in the
// reference.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/spear_btp_probe.h"
#include "btp_device.h"
#include "btp_launch.h"
#include "btp_staging.h"

namespace spear_btp {

namespace {

__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                   unsigned long long n16) {
  const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    dst[i] = src[i];
}

// Bandwidth probe with the operator's own access shape and cache policy and no arithmetic: every
// wavefront moves one 4 KiB slab (four 16-byte accesses per lane) with non-temporal loads and stores.
// kReads = 1: copy; kReads = 2: two inputs combined into one output, the backward kernel's mix.
template <int kReads>
__global__ __launch_bounds__(64 * kWaves) void stream_probe_kernel(const uint4* __restrict__ a,
                                                                   const uint4* __restrict__ b,
                                                                   uint4* __restrict__ dst, unsigned long long slabs) {
  const unsigned long long slab = (unsigned long long)blockIdx.x * kWaves + (threadIdx.x >> 6);
  if (slab >= slabs) return;
  const unsigned long long base = slab * 256 + (threadIdx.x & 63);
  uint4 q[4], r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    q[i] = stream_load16(a + base + 64 * i);
    if constexpr (kReads == 2) r[i] = stream_load16(b + base + 64 * i);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (kReads == 2) q[i] = make_uint4(q[i].x ^ r[i].x, q[i].y ^ r[i].y, q[i].z ^ r[i].z, q[i].w ^ r[i].w);
    stream_store16(dst + base + 64 * i, q[i]);
  }
}

// Other launch shapes for the same traffic, to show where the shape above stands (measured on MI355X: none
// of them is faster). kShape 1: two slabs per wavefront, every load issued before the first store (twice
// the bytes in flight per wavefront); 2: a loop over `iters` slabs per wavefront with the next slab's loads
// issued before the current slab's stores (a workgroup covers kWaves * iters consecutive slabs); 3: the
// same loop as a persistent grid striding over the buffer; 4: one 16-byte element per thread; 5 and 6: one
// direction only (reads without writes, writes without reads), which gives the two rates a mixed kernel's
// time is made of -- HBM serves reads and writes one after the other, so a kernel that reads R bytes and
// writes W bytes cannot finish before R / read rate + W / write rate; 7: shape 0 with a chain of 640 dependent
// FMAs between the loads and the stores (what a compute phase of the backward kernel's length costs even
// though the vector units are far from busy: every wavefront holds its slot that much longer).
template <int kReads, int kShape>
__global__ __launch_bounds__(64 * kWaves) void stream_probe_shape_kernel(const uint4* __restrict__ a,
                                                                         const uint4* __restrict__ b,
                                                                         uint4* __restrict__ dst,
                                                                         unsigned long long slabs, int iters) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  auto load = [&](unsigned long long slab, uint4 (&q)[4], uint4 (&r)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      q[i] = stream_load16(a + slab * 256 + lane + 64 * i);
      if constexpr (kReads == 2) r[i] = stream_load16(b + slab * 256 + lane + 64 * i);
    }
  };
  auto store = [&](unsigned long long slab, uint4 (&q)[4], const uint4 (&r)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (kReads == 2) q[i] = make_uint4(q[i].x ^ r[i].x, q[i].y ^ r[i].y, q[i].z ^ r[i].z, q[i].w ^ r[i].w);
      stream_store16(dst + slab * 256 + lane + 64 * i, q[i]);
    }
  };
  if constexpr (kShape == 1) {
    const unsigned long long s0 = (unsigned long long)blockIdx.x * kWaves * 2 + wave, s1 = s0 + kWaves;
    uint4 q0[4], r0[4], q1[4], r1[4];
    if (s0 < slabs) load(s0, q0, r0);
    if (s1 < slabs) load(s1, q1, r1);
    if (s0 < slabs) store(s0, q0, r0);
    if (s1 < slabs) store(s1, q1, r1);
  } else if constexpr (kShape == 2 || kShape == 3) {
    const unsigned long long step = kShape == 2 ? kWaves : (unsigned long long)gridDim.x * kWaves;
    unsigned long long slab = kShape == 2 ? (unsigned long long)blockIdx.x * kWaves * iters + wave
                                          : (unsigned long long)blockIdx.x * kWaves + wave;
    const unsigned long long end = kShape == 2 ? slab + step * iters : slabs;
    uint4 q[4], r[4], nq[4], nr[4];
    if (slab < slabs) load(slab, nq, nr);
    for (; slab < slabs && slab < end; slab += step) {
#pragma unroll
      for (int i = 0; i < 4; ++i) { q[i] = nq[i]; r[i] = nr[i]; }
      const unsigned long long next = slab + step;
      if (next < slabs && next < end) load(next, nq, nr);
      __builtin_amdgcn_sched_barrier(0);
      store(slab, q, r);
      __builtin_amdgcn_sched_barrier(0);
    }
  } else if constexpr (kShape == 5 || kShape == 6) {
    // one direction only, in the kernels' own shape: 5 reads the inputs and writes nothing (the store below
    // never happens for real data: it needs all-ones words), 6 writes `dst` and reads nothing
    const unsigned long long slab = (unsigned long long)blockIdx.x * kWaves + wave;
    if (slab >= slabs) return;
    uint4 q[4], r[4];
    if constexpr (kShape == 5) {
      load(slab, q, r);
      uint32_t all = 0xffffffffu;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        all &= q[i].x & q[i].y & q[i].z & q[i].w;
        if constexpr (kReads == 2) all &= r[i].x & r[i].y & r[i].z & r[i].w;
      }
      if (all == 0xffffffffu) stream_store16(dst + slab * 256 + lane, q[0]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        q[i] = make_uint4((uint32_t)slab, (uint32_t)lane, (uint32_t)i, 0u);
        stream_store16(dst + slab * 256 + lane + 64 * i, q[i]);
      }
    }
  } else if constexpr (kShape == 7) {
    // the kernels' own shape with arithmetic between the loads and the stores: a chain of 640 dependent FMAs,
    // about the backward kernel's instruction count, whose result flips one bit of the output's last word
    const unsigned long long slab = (unsigned long long)blockIdx.x * kWaves + wave;
    if (slab >= slabs) return;
    uint4 q[4], r[4];
    load(slab, q, r);
    float acc = __uint_as_float(q[0].x & 0x3fffffffu);
#pragma unroll 1
    for (int s = 0; s < 80; ++s) {
#pragma unroll
      for (int u = 0; u < 8; ++u) acc = __builtin_fmaf(acc, 0.999f, 0.001f);
    }
    q[3].w ^= __float_as_uint(acc) & 1u;
    store(slab, q, r);
  } else {
    static_assert(kShape == 4, "unknown probe shape");
    const unsigned long long i = (unsigned long long)blockIdx.x * (64 * kWaves) + threadIdx.x;
    if (i < slabs * 256) {
      uint4 q = stream_load16(a + i);
      if constexpr (kReads == 2) {
        const uint4 r = stream_load16(b + i);
        q = make_uint4(q.x ^ r.x, q.y ^ r.y, q.z ^ r.z, q.w ^ r.w);
      }
      stream_store16(dst + i, q);
    }
  }
}

// The probe for kernels with more streams: kIn inputs combined into kOut identical outputs, every tensor `slabs`
// pieces of 4 KiB, one piece per wavefront and tensor, non-temporal 16-byte accesses (the fused layer kernels read
// 3 or 4 big tensors and write 1 or 3). kSpin > 0 puts 8 * kSpin dependent FMAs between the loads and the stores;
// their result flips the lowest bit of every output's last word.
struct ProbeMixPtrs {
  const uint4* in[4];
  uint4* out[3];
};
template <int kIn, int kOut, int kSpin>
__global__ __launch_bounds__(64 * kWaves) void stream_probe_mix_kernel(ProbeMixPtrs p, unsigned long long slabs) {
  const unsigned long long slab = (unsigned long long)blockIdx.x * kWaves + (threadIdx.x >> 6);
  if (slab >= slabs) return;
  const unsigned long long base = slab * 256 + (threadIdx.x & 63);
  uint4 q[kIn][4];
#pragma unroll
  for (int t = 0; t < kIn; ++t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) q[t][i] = stream_load16(p.in[t] + base + 64 * i);
  }
  float acc = __uint_as_float(q[0][0].x & 0x3fffffffu);
#pragma unroll 1
  for (int s = 0; s < kSpin; ++s) {
#pragma unroll
    for (int u = 0; u < 8; ++u) acc = __builtin_fmaf(acc, 0.999f, 0.001f);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint4 o = q[0][i];
#pragma unroll
    for (int t = 1; t < kIn; ++t) o = make_uint4(o.x ^ q[t][i].x, o.y ^ q[t][i].y, o.z ^ q[t][i].z, o.w ^ q[t][i].w);
    if (kSpin > 0 && i == 3) o.w ^= __float_as_uint(acc) & 1u;
#pragma unroll
    for (int t = 0; t < kOut; ++t) stream_store16(p.out[t] + base + 64 * i, o);
  }
}

}  // namespace

hipError_t stream_probe(const void* a, const void* b, void* dst, unsigned long long bytes, hipStream_t s) {
  const unsigned long long slabs = bytes / 4096;
  if (slabs == 0) return hipSuccess;
  const unsigned blocks = (unsigned)((slabs + kWaves - 1) / kWaves);
  if (b == nullptr)
    hipLaunchKernelGGL(stream_probe_kernel<1>, dim3(blocks), dim3(64 * kWaves), 0, s, static_cast<const uint4*>(a),
                       static_cast<const uint4*>(nullptr), static_cast<uint4*>(dst), slabs);
  else
    hipLaunchKernelGGL(stream_probe_kernel<2>, dim3(blocks), dim3(64 * kWaves), 0, s, static_cast<const uint4*>(a),
                       static_cast<const uint4*>(b), static_cast<uint4*>(dst), slabs);
  return hipGetLastError();
}

namespace {
template <int kReads>
void launch_probe_shape(const void* a, const void* b, void* dst, unsigned long long slabs, int shape, hipStream_t s) {
  const auto* pa = static_cast<const uint4*>(a);
  const auto* pb = static_cast<const uint4*>(b);
  auto* pd = static_cast<uint4*>(dst);
  const dim3 wg(64 * kWaves);
  auto blocks_for = [&](unsigned long long per) { return dim3((unsigned)((slabs + per - 1) / per)); };
  constexpr int kLoopIters = 4;
  switch (shape) {
    case 1: hipLaunchKernelGGL((stream_probe_shape_kernel<kReads, 1>), blocks_for(2 * kWaves), wg, 0, s, pa, pb, pd, slabs, 2); break;
    case 2: hipLaunchKernelGGL((stream_probe_shape_kernel<kReads, 2>), blocks_for(kLoopIters * kWaves), wg, 0, s, pa, pb, pd, slabs, kLoopIters); break;
    case 3: {
      const unsigned long long want = (slabs + kWaves - 1) / kWaves;
      hipLaunchKernelGGL((stream_probe_shape_kernel<kReads, 3>), dim3((unsigned)(want < 2048 ? want : 2048)), wg, 0, s, pa, pb, pd, slabs, 0);
      break;
    }
    case 5: hipLaunchKernelGGL((stream_probe_shape_kernel<kReads, 5>), blocks_for(kWaves), wg, 0, s, pa, pb, pd, slabs, 1); break;
    case 6: hipLaunchKernelGGL((stream_probe_shape_kernel<kReads, 6>), blocks_for(kWaves), wg, 0, s, pa, pb, pd, slabs, 1); break;
    case 7: hipLaunchKernelGGL((stream_probe_shape_kernel<kReads, 7>), blocks_for(kWaves), wg, 0, s, pa, pb, pd, slabs, 1); break;
    default: hipLaunchKernelGGL((stream_probe_shape_kernel<kReads, 4>), blocks_for(1), wg, 0, s, pa, pb, pd, slabs, 1); break;
  }
}
}  // namespace

hipError_t stream_probe_shape(const void* a, const void* b, void* dst, unsigned long long bytes, int shape, hipStream_t s) {
  if (shape == 0) return stream_probe(a, b, dst, bytes, s);
  const unsigned long long slabs = bytes / 4096;
  if (slabs == 0) return hipSuccess;
  if (b == nullptr) launch_probe_shape<1>(a, b, dst, slabs, shape, s);
  else launch_probe_shape<2>(a, b, dst, slabs, shape, s);
  return hipGetLastError();
}

hipError_t stream_probe_mix(const void* const* src, int n_src, void* const* dst, int n_dst, unsigned long long bytes,
                            bool compute, hipStream_t s) {
  const unsigned long long slabs = bytes / 4096;
  if (slabs == 0) return hipSuccess;
  ProbeMixPtrs p{};
  for (int i = 0; i < n_src; ++i) p.in[i] = static_cast<const uint4*>(src[i]);
  for (int i = 0; i < n_dst; ++i) p.out[i] = static_cast<uint4*>(dst[i]);
  const dim3 grid((unsigned)((slabs + kWaves - 1) / kWaves)), wg(64 * kWaves);
  if (n_src == 4 && n_dst == 3) {
    if (compute) hipLaunchKernelGGL((stream_probe_mix_kernel<4, 3, 160>), grid, wg, 0, s, p, slabs);
    else hipLaunchKernelGGL((stream_probe_mix_kernel<4, 3, 0>), grid, wg, 0, s, p, slabs);
  } else if (n_src == 3 && n_dst == 1) {
    if (compute) hipLaunchKernelGGL((stream_probe_mix_kernel<3, 1, 80>), grid, wg, 0, s, p, slabs);
    else hipLaunchKernelGGL((stream_probe_mix_kernel<3, 1, 0>), grid, wg, 0, s, p, slabs);
  } else if (n_src == 1 && n_dst == 2) {
    if (compute) hipLaunchKernelGGL((stream_probe_mix_kernel<1, 2, 40>), grid, wg, 0, s, p, slabs);
    else hipLaunchKernelGGL((stream_probe_mix_kernel<1, 2, 0>), grid, wg, 0, s, p, slabs);
  } else {
    return hipErrorInvalidValue;  // the caller has checked
  }
  return hipGetLastError();
}

hipError_t device_copy(const void* src, void* dst, unsigned long long bytes, hipStream_t s) {
  const unsigned long long n16 = bytes / 16;
  if (n16 == 0) return hipSuccess;
  unsigned long long want = (n16 + 255) / 256;
  const unsigned blocks = (unsigned)(want < 256ull * 32 ? want : 256ull * 32);
  hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const uint4*>(src),
                     static_cast<uint4*>(dst), n16);
  return hipGetLastError();
}

}  // namespace spear_btp

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

extern "C" {

int spear_btp_copy(const void* src, void* dst, unsigned long long bytes, void* stream) {
  spear_btp::clear_error();
  if (!src || !dst) return spear_btp::report_error(SPEAR_BTP_ENULL, "spear_btp_copy: NULL pointer");
  if (bytes % 16 != 0 || !aligned16(src) || !aligned16(dst))
    return spear_btp::report_error(SPEAR_BTP_EINVAL, "spear_btp_copy: size and pointers must be multiples of 16 bytes");
  const hipError_t err = spear_btp::device_copy(src, dst, bytes, static_cast<hipStream_t>(stream));
  if (err != hipSuccess) return spear_btp::report_error(SPEAR_BTP_ELAUNCH, "spear_btp_copy: launch failed: %s", hipGetErrorString(err));
  return 0;
}

int spear_btp_stream_probe(const void* src_a, const void* src_b, void* dst, unsigned long long bytes, void* stream) {
  spear_btp::clear_error();
  if (!src_a || !dst) return spear_btp::report_error(SPEAR_BTP_ENULL, "spear_btp_stream_probe: NULL pointer");
  if (bytes % 4096 != 0 || !aligned16(src_a) || !aligned16(src_b) || !aligned16(dst))
    return spear_btp::report_error(SPEAR_BTP_EINVAL, "spear_btp_stream_probe: size must be a multiple of 4096, pointers of 16 bytes");
  const hipError_t err = spear_btp::stream_probe(src_a, src_b, dst, bytes, static_cast<hipStream_t>(stream));
  if (err != hipSuccess)
    return spear_btp::report_error(SPEAR_BTP_ELAUNCH, "spear_btp_stream_probe: launch failed: %s", hipGetErrorString(err));
  return 0;
}

int spear_btp_stream_probe_shape(const void* src_a, const void* src_b, void* dst, unsigned long long bytes, int shape,
                                 void* stream) {
  spear_btp::clear_error();
  if (!src_a || !dst) return spear_btp::report_error(SPEAR_BTP_ENULL, "spear_btp_stream_probe_shape: NULL pointer");
  if (bytes % 4096 != 0 || !aligned16(src_a) || !aligned16(src_b) || !aligned16(dst))
    return spear_btp::report_error(SPEAR_BTP_EINVAL, "spear_btp_stream_probe_shape: size must be a multiple of 4096, pointers of 16 bytes");
  if (shape < 0 || shape >= SPEAR_BTP_PROBE_SHAPES)
    return spear_btp::report_error(SPEAR_BTP_EINVAL, "spear_btp_stream_probe_shape: shape must be 0..%d (got %d)", SPEAR_BTP_PROBE_SHAPES - 1, shape);
  const hipError_t err = spear_btp::stream_probe_shape(src_a, src_b, dst, bytes, shape, static_cast<hipStream_t>(stream));
  if (err != hipSuccess)
    return spear_btp::report_error(SPEAR_BTP_ELAUNCH, "spear_btp_stream_probe_shape: launch failed: %s", hipGetErrorString(err));
  return 0;
}

int spear_btp_stream_probe_mix(const void* const* src, int n_src, void* const* dst, int n_dst, unsigned long long bytes,
                               int compute, void* stream) {
  spear_btp::clear_error();
  const char* who = "spear_btp_stream_probe_mix";
  if (!src || !dst) return spear_btp::report_error(SPEAR_BTP_ENULL, "%s: NULL pointer", who);
  if (!((n_src == 3 && n_dst == 1) || (n_src == 4 && n_dst == 3) || (n_src == 1 && n_dst == 2)))
    return spear_btp::report_error(SPEAR_BTP_EINVAL, "%s: (n_src, n_dst) must be (3, 1), (4, 3) or (1, 2) (got %d, %d)", who, n_src, n_dst);
  if (bytes % 4096 != 0) return spear_btp::report_error(SPEAR_BTP_EINVAL, "%s: size must be a multiple of 4096", who);
  for (int i = 0; i < n_src; ++i)
    if (!src[i] || !aligned16(src[i])) return spear_btp::report_error(SPEAR_BTP_EINVAL, "%s: every tensor pointer must be set and 16-byte aligned", who);
  for (int i = 0; i < n_dst; ++i)
    if (!dst[i] || !aligned16(dst[i])) return spear_btp::report_error(SPEAR_BTP_EINVAL, "%s: every tensor pointer must be set and 16-byte aligned", who);
  const hipError_t err = spear_btp::stream_probe_mix(src, n_src, dst, n_dst, bytes, compute != 0, static_cast<hipStream_t>(stream));
  if (err != hipSuccess) return spear_btp::report_error(SPEAR_BTP_ELAUNCH, "%s: launch failed: %s", who, hipGetErrorString(err));
  return 0;
}

}  // extern "C"
