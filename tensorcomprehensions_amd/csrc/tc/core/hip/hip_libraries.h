// Device-side helper library prepended to every generated kernel, as source text for hipRTC.
//
// Role of tc/core/cuda/cuda_libraries.h:33-285 in the reference, rewritten for 64-lane
// wavefronts: floor-division helpers for index arithmetic, reduction operators with their
// identities, and a block reduction "along x" that replaces the CUB-based CubReduceAlongX
// (:214-285).  The reduction is hand-written: DPP butterflies inside 16-lane rows, lane reads
// across rows, LDS across wavefronts.
#pragma once
#include <string>

namespace tc {
namespace hip {

constexpr const char* kDeviceTypes = R"HIP(
typedef long long int64;
typedef unsigned long long uint64;
namespace __tc {
typedef float floatx4 __attribute__((ext_vector_type(4)));
// same vector read through a pointer that is only element-aligned
typedef float floatx4u __attribute__((ext_vector_type(4), aligned(4)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx4u __attribute__((ext_vector_type(4), aligned(2)));
}
)HIP";

// Halide-style integer semantics for / and % in subscripts (round toward -infinity),
// cf. floord in tc/core/cuda/cuda_libraries.h:61-66.
constexpr const char* kDeviceIndexHelpers = R"HIP(
namespace __tc {
template <typename T> __device__ __forceinline__ T floordiv(T n, T d) {
  T q = n / d;
  return ((n % d != 0) && ((n < 0) != (d < 0))) ? q - 1 : q;
}
template <typename T> __device__ __forceinline__ T floormod(T n, T d) { return n - floordiv(n, d) * d; }
// Store of element `index` of the tensor behind buffer descriptor `rs` with device-scope
// write-through (cache policy sc1 = 16): the value goes on to memory instead of staying dirty in
// the L2 until the end of the kernel.  An offset past the end of the buffer is dropped.
template <typename T> __device__ __forceinline__ void storeThrough(__amdgpu_buffer_rsrc_t rs, int index, T v) {
  typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
  if constexpr (sizeof(T) == 8) {
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(uintx2, v), rs, index * 8, 0, 16);
  } else if constexpr (sizeof(T) == 4) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rs, index * 4, 0, 16);
  } else if constexpr (sizeof(T) == 2) {
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), rs, index * 2, 0, 16);
  } else {
    __builtin_amdgcn_raw_buffer_store_b8(__builtin_bit_cast(unsigned char, v), rs, index, 0, 16);
  }
}
// Partial sum of one block into an element other blocks add to as well (device scope, no order).
template <typename T> __device__ __forceinline__ void atomicAccumulate(T* p, T v) {
  __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The same for any other combining operator (product, minimum, maximum) of a 32- or 64-bit
// element: compare-and-swap on the bit pattern until the combined value is in place.
template <typename Op, typename T> __device__ __forceinline__ void atomicCombine(T* p, T v) {
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32- or 64-bit elements");
  if constexpr (sizeof(T) == 4) {
    unsigned* q = reinterpret_cast<unsigned*>(p);
    unsigned seen = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while (true) {
      const unsigned want = __builtin_bit_cast(unsigned, Op::apply(__builtin_bit_cast(T, seen), v));
      if (want == seen) break;
      if (__hip_atomic_compare_exchange_strong(q, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
    }
  } else {
    unsigned long long* q = reinterpret_cast<unsigned long long*>(p);
    unsigned long long seen = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while (true) {
      const unsigned long long want = __builtin_bit_cast(unsigned long long, Op::apply(__builtin_bit_cast(T, seen), v));
      if (want == seen) break;
      if (__hip_atomic_compare_exchange_strong(q, &seen, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
    }
  }
}
// Value of lane ^ MASK for MASK = 16 or 32, through v_permlane16_swap_b32 / v_permlane32_swap_b32
// (gfx950: rows, respectively halves, of two registers change places in the vector ALU; a
// ds_bpermute would go through the LDS crossbar and its wait counter).  With both operands equal
// to u the instruction leaves {even rows | low half} of u everywhere in the first result and
// {odd rows | high half} in the second: a lane takes the one its partner lives in.
template <int MASK> __device__ __forceinline__ unsigned laneXor32(unsigned u) {
  static_assert(MASK == 16 || MASK == 32, "partner across 16-lane rows or across the halves of a wavefront");
  const unsigned lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  if constexpr (MASK == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return (lane & 16u) ? r[0] : r[1];
  } else {
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return (lane & 32u) ? r[0] : r[1];
  }
}
template <int MASK> __device__ __forceinline__ float laneXor32(float v) {
  return __builtin_bit_cast(float, laneXor32<MASK>(__builtin_bit_cast(unsigned, v)));
}
template <typename T> __device__ __forceinline__ T tmin(T a, T b) { return a < b ? a : b; }
template <typename T> __device__ __forceinline__ T tmax(T a, T b) { return a > b ? a : b; }
__device__ __forceinline__ float tmin(float a, float b) { return fminf(a, b); }
__device__ __forceinline__ float tmax(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ _Float16 tmin(_Float16 a, _Float16 b) { return (_Float16)fminf((float)a, (float)b); }
__device__ __forceinline__ _Float16 tmax(_Float16 a, _Float16 b) { return (_Float16)fmaxf((float)a, (float)b); }
__device__ __forceinline__ double tmin(double a, double b) { return fmin(a, b); }
__device__ __forceinline__ double tmax(double a, double b) { return fmax(a, b); }
} // namespace __tc
)HIP";

// Wave64 reduction library.
//   __tc::OpSum/OpProd/OpMin/OpMax<T>      operator + identity
//   __tc::waveAllReduce<Op, WIDTH>(v)      all-reduce over aligned groups of WIDTH lanes
//                                          (WIDTH a power of two, 2..64)
//   __tc::blockAllReduceX<Op, BX, BY, BZ>(v, scratch)
//        reduces v over threadIdx.x separately for every (threadIdx.y, threadIdx.z) and
//        returns the result to every thread of the row.  `scratch` is LDS of
//        __tc::reduceScratchElems(BX, BY, BZ) elements; the call contains block barriers, so
//        every thread of the block must reach it.
constexpr const char* kDeviceReductions = R"HIP(
namespace __tc {
template <typename T> struct OpSum  { static __device__ __forceinline__ T apply(T a, T b) { return a + b; } };
template <typename T> struct OpProd { static __device__ __forceinline__ T apply(T a, T b) { return a * b; } };
template <typename T> struct OpMin  { static __device__ __forceinline__ T apply(T a, T b) { return tmin(a, b); } };
template <typename T> struct OpMax  { static __device__ __forceinline__ T apply(T a, T b) { return tmax(a, b); } };

// lane exchange through the DPP network (no LDS traffic); CTRL is a GFX9 dpp_ctrl code.  Any
// arithmetic type of up to 64 bits: 64-bit values move as two 32-bit halves, narrower ones
// widened to one.
template <int CTRL> __device__ __forceinline__ int dppMov32(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xf, 0xf, false);
}
template <int CTRL, typename T> __device__ __forceinline__ T dppMov(T v) {
  static_assert(sizeof(T) <= 8, "lane exchange of at most 64 bits");
  if constexpr (sizeof(T) == 8) {
    const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
    const unsigned lo = (unsigned)dppMov32<CTRL>((int)(unsigned)(b & 0xffffffffULL));
    const unsigned hi = (unsigned)dppMov32<CTRL>((int)(unsigned)(b >> 32));
    return __builtin_bit_cast(T, ((unsigned long long)hi << 32) | lo);
  } else if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, dppMov32<CTRL>(__builtin_bit_cast(int, v)));
  } else if constexpr (sizeof(T) == 2) {
    // by bit pattern: the element may be a half
    return __builtin_bit_cast(T, (unsigned short)dppMov32<CTRL>((int)__builtin_bit_cast(unsigned short, v)));
  } else {
    return (T)dppMov32<CTRL>((int)v);
  }
}
// exchange with lane ^ MASK (16 or 32) across the 16-lane rows of a wavefront
template <int MASK, typename T> __device__ __forceinline__ T laneXor(T v) {
  if constexpr (sizeof(T) == 8) {
    const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
    const unsigned lo = laneXor32<MASK>((unsigned)(b & 0xffffffffULL));
    const unsigned hi = laneXor32<MASK>((unsigned)(b >> 32));
    return __builtin_bit_cast(T, ((unsigned long long)hi << 32) | lo);
  } else if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, laneXor32<MASK>(__builtin_bit_cast(unsigned, v)));
  } else if constexpr (sizeof(T) == 2) {
    return __builtin_bit_cast(T, (unsigned short)laneXor32<MASK>((unsigned)__builtin_bit_cast(unsigned short, v)));
  } else {
    return (T)(int)laneXor32<MASK>((unsigned)(int)v);
  }
}

// 0xB1 = quad_perm[1,0,3,2] (lane^1), 0x4E = quad_perm[2,3,0,1] (lane^2),
// 0x141 = row_half_mirror (i <-> 7-i), 0x140 = row_mirror (i <-> 15-i).
template <typename Op, int WIDTH, typename T> __device__ __forceinline__ T waveAllReduce(T v) {
  static_assert(WIDTH >= 1 && WIDTH <= 64 && (WIDTH & (WIDTH - 1)) == 0, "power of two up to 64");
  if constexpr (WIDTH >= 2) v = Op::apply(v, dppMov<0xB1>(v));
  if constexpr (WIDTH >= 4) v = Op::apply(v, dppMov<0x4E>(v));
  if constexpr (WIDTH >= 8) v = Op::apply(v, dppMov<0x141>(v));
  if constexpr (WIDTH >= 16) v = Op::apply(v, dppMov<0x140>(v));
  if constexpr (WIDTH >= 32) v = Op::apply(v, laneXor<16>(v));
  if constexpr (WIDTH >= 64) v = Op::apply(v, laneXor<32>(v));
  return v;
}

__host__ __device__ constexpr int reduceScratchElems(int bx, int by, int bz) {
  return ((bx & (bx - 1)) == 0 && bx <= 64) ? 1 : (bx % 64 == 0 ? (bx / 64) * by * bz : bx * by * bz);
}

// Completes the value here: the combine chain of one reduction is finished before the next
// barrier instead of being deferred, which bounds the values in flight when many reductions are
// unrolled back to back (hundreds of deferred LDS reads otherwise end up spilled).
template <typename T> __device__ __forceinline__ void settle(T&) {}
__device__ __forceinline__ void settle(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void settle(double& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void settle(int& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void settle(unsigned& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void settle(long long& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void settle(unsigned long long& v) { asm volatile("" : "+v"(v)); }

template <typename Op, int BX, int BY, int BZ, typename T>
__device__ __forceinline__ T blockAllReduceX(T v, T* scratch) {
  if constexpr (BX == 1) {
    return v;
  } else if constexpr ((BX & (BX - 1)) == 0 && BX <= 64) {
    // a row of BX threads is an aligned lane group of one wavefront
    // (linear thread id = x + BX * (y + BY * z), BX divides 64)
    return waveAllReduce<Op, BX>(v);
  } else if constexpr (BX % 64 == 0) {
    // every wavefront lies inside one row: wave reduce, then combine BX/64 partials through LDS
    const int row = threadIdx.y + BY * threadIdx.z;
    constexpr int W = BX / 64;
    v = waveAllReduce<Op, 64>(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[row * W + (threadIdx.x >> 6)] = v;
    __syncthreads();
    T r = scratch[row * W];
#pragma unroll
    for (int w = 1; w < W; ++w) r = Op::apply(r, scratch[row * W + w]);
    settle(r);
    return r;
  } else {
    // any other row width: rows straddle wavefronts, go through LDS.  Two levels: the first G
    // threads of a row each combine a chunk of C values, then every thread combines the G
    // partial results (C + G reads per thread instead of BX: 22 instead of 111 for a row of 111).
    const int row = threadIdx.y + BY * threadIdx.z;
    constexpr int C = BX <= 16 ? BX : (BX <= 64 ? 8 : 16);
    constexpr int G = (BX + C - 1) / C;
    __syncthreads();
    scratch[row * BX + threadIdx.x] = v;
    __syncthreads();
    if constexpr (G > 1) {
      T part = v;
      if (threadIdx.x < G) {
        const int first = threadIdx.x * C;
        part = scratch[row * BX + first];
#pragma unroll
        for (int i = 1; i < C; ++i) {
          if (first + i < BX) part = Op::apply(part, scratch[row * BX + first + i]);
        }
      }
      __syncthreads();
      if (threadIdx.x < G) scratch[row * BX + threadIdx.x] = part;
      __syncthreads();
    }
    T r = scratch[row * BX];
#pragma unroll
    for (int g = 1; g < G; ++g) r = Op::apply(r, scratch[row * BX + g]);
    if constexpr (G == 1) {
#pragma unroll
      for (int x = 1; x < BX; ++x) r = Op::apply(r, scratch[row * BX + x]);
    }
    settle(r);
    return r;
  }
}
} // namespace __tc
)HIP";

inline std::string deviceLibrary(bool withReductions) {
  std::string s = std::string(kDeviceTypes) + kDeviceIndexHelpers;
  if (withReductions) {
    s += kDeviceReductions;
  }
  return s;
}

} // namespace hip
} // namespace tc
