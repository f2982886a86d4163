// Device-side building blocks for gfx950 (CDNA4): buffer resources, direct global->LDS loads,
// MFMA wrappers per element type, and fp32 -> 16-bit round-to-nearest-even conversion.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355 {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

// Element-type tags.  kBytes = bytes per element; kSliceChunks = 16-byte chunks of one operand
// row that a single lane feeds into one 32x32 MFMA (1 for 16-bit types: 8 elements; 2 for fp8:
// 32 elements).
struct BF16 { static constexpr int kBytes = 2; static constexpr int kSliceChunks = 1; };
struct F16  { static constexpr int kBytes = 2; static constexpr int kSliceChunks = 1; };
struct E4M3 { static constexpr int kBytes = 1; static constexpr int kSliceChunks = 2; };
// e4m3 elements that carry one E8M0 scale per 32 consecutive elements of K (OCP MX block scaling).
struct MxE4M3 : E4M3 {};

// Raw (unstructured) buffer descriptor over [base, base+bytes): loads beyond `bytes` return 0,
// which is how ragged tile edges are handled.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_raw_buffer(const void* base, uint32_t bytes) {
  // The descriptor must live in scalar registers.  The operands are wave-uniform by
  // construction; readfirstlane makes that visible to the compiler (64-bit address arithmetic
  // is done on the vector ALU and would otherwise drag the descriptor into vector registers).
  const uint64_t p = (uint64_t)base;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)p);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(p >> 32));
  void* q = (void*)(((uint64_t)hi << 32) | lo);
  return __builtin_amdgcn_make_buffer_rsrc(q, 0, (int)__builtin_amdgcn_readfirstlane(bytes), 0x00020000);
}

// One wave copies 64 x 16 B from global memory straight into LDS.  Lane l's 16 bytes come from
// buffer offset voffset(l) + soffset and land at LDS byte address lds_base + 16*l (lds_base is
// wave-uniform).  Completion is tracked by the wave's vmcnt counter; the compiler does not see
// the LDS write, so callers order it with wait_vmcnt<N>() and a workgroup barrier.
__device__ __forceinline__ void dma_16B_to_lds(uint32_t lds_base, uint32_t voffset,
                                               __amdgpu_buffer_rsrc_t rsrc, uint32_t soffset) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen lds"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(voffset), "s"(rsrc),
        "s"(__builtin_amdgcn_readfirstlane(soffset))
      : "memory");
}

// The same with 4 bytes per lane: lane l's dword lands at LDS byte address lds_base + 4*l.
__device__ __forceinline__ void dma_4B_to_lds(uint32_t lds_base, uint32_t voffset,
                                              __amdgpu_buffer_rsrc_t rsrc, uint32_t soffset) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "buffer_load_dword %1, %2, %3 offen lds"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(voffset), "s"(rsrc),
        "s"(__builtin_amdgcn_readfirstlane(soffset))
      : "memory");
}

// The same copy with the LDS base given as a scalar register plus a compile-time constant, folded
// into the one instruction that writes M0 (it also writes SCC).
template <uint32_t kLdsAdd>
__device__ __forceinline__ void dma_16B_to_lds_at(uint32_t lds_base, uint32_t voffset,
                                                  __amdgpu_buffer_rsrc_t rsrc, uint32_t soffset) {
  asm volatile(
      "s_add_u32 m0, %0, %4\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen lds"
      :
      : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(voffset), "s"(rsrc),
        "s"(__builtin_amdgcn_readfirstlane(soffset)), "n"(kLdsAdd)
      : "memory", "scc");
}

// 8 bytes per lane from buffer offset voffset(l) + soffset into a register pair, WITHOUT the
// compiler knowing that the result arrives later: the caller must pass the pair through
// wait_vmcnt_for<N>() (N = vector-memory instructions issued after this one) before its first use,
// and must check in the generated code that the pair is not copied in between.
// MI355_MX_SYNC_SCALES: the fallback the build switches to when that check of the generated code
// fails (a different compiler may copy such a register): the load then waits for itself, and with
// it for every copy in flight, which costs time in every k-step but needs no promise from the
// register allocator.
__device__ __forceinline__ void load_8B_async(u32x2& dst, __amdgpu_buffer_rsrc_t rsrc, uint32_t voffset,
                                              uint32_t soffset) {
#ifdef MI355_MX_SYNC_SCALES
  asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen\n\ts_waitcnt vmcnt(0)"
#else
  asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen"
#endif
               : "=v"(dst)
               : "v"(voffset), "s"(rsrc), "s"(__builtin_amdgcn_readfirstlane(soffset))
               : "memory");
}

// The two halves of dma_16B_to_lds_at as separate statements, so that other instructions can sit
// between the write of M0 and the copy that uses it.
template <uint32_t kLdsAdd>
__device__ __forceinline__ void dma_set_lds_base(uint32_t lds_base) {
  asm volatile("s_add_u32 m0, %0, %1" ::"s"(__builtin_amdgcn_readfirstlane(lds_base)), "n"(kLdsAdd) : "scc");
}
__device__ __forceinline__ void dma_16B_to_lds_base_set(uint32_t voffset, __amdgpu_buffer_rsrc_t rsrc, uint32_t soffset) {
  asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(voffset), "s"(rsrc),
               "s"(__builtin_amdgcn_readfirstlane(soffset))
               : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// The same wait, naming the registers whose asynchronous loads it completes.
template <int N>
__device__ __forceinline__ void wait_vmcnt_for(u32x2& a, u32x2& b) {
  asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}
__device__ __forceinline__ void wait_lgkmcnt0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)p;
}

// Store data and the registers that hold it.  A vector-memory store of more than 8 bytes per lane
// reads its data registers over several cycles after it has issued, and the ISA asks for idle wait
// states between such a store and the next write of those registers.  The compiler provides them
// only for stores without a scalar offset register; the stores here have one.  With nothing in
// between, a few lanes of a store's first data register were seen to carry the NEXT store's value.
// So the code keeps the hazard from arising instead of waiting it out: the data registers of store
// n stay live, untouched, until the data of store n + 2 is complete (hold_previous names the new
// data and that of the two stores before it in one empty assembly statement, which the compiler
// can neither move in front of the conversion that produces the new data nor behind the store that
// consumes it, and a scheduling barrier behind every store keeps the next conversion from being
// hoisted above it), so the conversions of blocks n + 1 and n + 2 cannot be given the registers of
// store n, and three register sets rotate.  The first write into the registers of store n is then
// two whole conversions away (ten to thirty instructions each, depending on the kernel).
// check_async_loads.check_hazard_distances verifies exactly that in the generated assembly of every
// build: no write of a store's data registers within 12 wait states, on any path.
template <class V>
__device__ __forceinline__ void hold_previous(V& current, const V& previous, const V& before) {
  asm volatile("" : "+v"(current) : "v"(previous), "v"(before));
}
// Where no conversion follows a store -- the last store of a tile, and the fp32 partial tiles of a
// K split, whose data is the accumulator registers themselves -- the data registers are held over
// idle wait states instead: the wait states the ISA asks for, counted, not a delay tuned by trial.
template <class V>
__device__ __forceinline__ void hold_last(const V& last) {
  asm volatile("s_nop 11" ::"v"(last) : "memory");
}

// Four fp32 -> four 16-bit values (round to nearest even), packed into 8 bytes.
template <class OutT> struct Pack4;
template <> struct Pack4<BF16> {
  static __device__ __forceinline__ u32x2 run(float a, float b, float c, float d) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf2;
    typedef __attribute__((ext_vector_type(2))) float f2;
    bf2 lo = __builtin_convertvector((f2){a, b}, bf2);
    bf2 hi = __builtin_convertvector((f2){c, d}, bf2);
    return (u32x2){__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi)};
  }
  static __device__ __forceinline__ uint16_t one(float a) {
    return __builtin_bit_cast(uint16_t, (__bf16)a);
  }
};
template <> struct Pack4<F16> {
  static __device__ __forceinline__ u32x2 run(float a, float b, float c, float d) {
    typedef __attribute__((ext_vector_type(2))) _Float16 h2;
    typedef __attribute__((ext_vector_type(2))) float f2;
    h2 lo = __builtin_convertvector((f2){a, b}, h2);
    h2 hi = __builtin_convertvector((f2){c, d}, h2);
    return (u32x2){__builtin_bit_cast(unsigned, lo), __builtin_bit_cast(unsigned, hi)};
  }
  static __device__ __forceinline__ uint16_t one(float a) {
    return __builtin_bit_cast(uint16_t, (_Float16)a);
  }
};

// Element -> fp32 for the one-thread-per-output kernel.
template <class T> struct Decode;
template <> struct Decode<BF16> {
  static __device__ __forceinline__ float run(const void* p, int64_t i) {
    uint32_t u = ((const uint16_t*)p)[i];
    return __builtin_bit_cast(float, u << 16);
  }
};
template <> struct Decode<F16> {
  static __device__ __forceinline__ float run(const void* p, int64_t i) {
    return (float)((const _Float16*)p)[i];
  }
};
template <> struct Decode<E4M3> {
  // OCP e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities; S.1111.111 = NaN.
  static __device__ __forceinline__ float run(const void* p, int64_t i) {
    uint32_t b = ((const uint8_t*)p)[i];
    uint32_t s = b >> 7, e = (b >> 3) & 15, m = b & 7;
    float v;
    if (e == 0) v = (float)m * 0.001953125f;                 // m * 2^-9 (subnormal)
    else if (e == 15 && m == 7) v = __builtin_nanf("");
    else v = __builtin_bit_cast(float, ((e + 120u) << 23) | (m << 20));
    return s ? -v : v;
  }
};

}  // namespace mi355
