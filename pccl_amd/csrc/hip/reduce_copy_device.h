// reduce_copy_device.h -- gfx950 device code shared by the direct-launch kernels
// and the persistent work-queue kernel.
//
// One lane moves 16-byte packs (the widest packs of the reference's
// include/plugins/cuda_executor/utils/vector_datatype.h:64-71: i32x4, f32x4,
// f16x8, bf16x8), so a 64-lane wavefront covers 1 KiB of every stream per
// load/store instruction.  The N-input fold replaces the switch-side
// multimem.ld_reduce of include/plugins/cuda_executor/utils/multimem.h:12-59
// with N explicit loads and a left fold in registers; the store to every
// output replaces multimem.st (multimem.h:61-102).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "pccl_hip.h"

namespace pccl_dev {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// Same 16 bytes, but the compiler may only assume the stated alignment.  The
// HSA ABI runs gfx9 in unaligned access mode, so these still compile to one
// global_load_dwordx4 / global_store_dwordx4.
typedef u32x4 u32x4_a8 __attribute__((aligned(8)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
typedef u32x4 u32x4_a1 __attribute__((aligned(1)));

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kBlock = 256;  // 4 wavefronts, one per SIMD of a compute unit

__device__ __forceinline__ float as_f32(unsigned int u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ unsigned int as_u32(float f) { return __builtin_bit_cast(unsigned int, f); }

// ---- fold operators: a is the accumulator, b the next input ----------------
// f: binary32 accumulator, d: binary64, i: int32 in two's complement, u: uint32
struct OpSum {
  static __device__ __forceinline__ float f(float a, float b) { return a + b; }
  static __device__ __forceinline__ double d(double a, double b) { return a + b; }
  static __device__ __forceinline__ unsigned int i(unsigned int a, unsigned int b) { return a + b; }
  static __device__ __forceinline__ unsigned int u(unsigned int a, unsigned int b) { return a + b; }
};
struct OpProd {
  static __device__ __forceinline__ float f(float a, float b) { return a * b; }
  static __device__ __forceinline__ double d(double a, double b) { return a * b; }
  static __device__ __forceinline__ unsigned int i(unsigned int a, unsigned int b) { return a * b; }
  static __device__ __forceinline__ unsigned int u(unsigned int a, unsigned int b) { return a * b; }
};
struct OpMin {
  static __device__ __forceinline__ float f(float a, float b) { return b < a ? b : a; }
  static __device__ __forceinline__ double d(double a, double b) { return b < a ? b : a; }
  static __device__ __forceinline__ unsigned int i(unsigned int a, unsigned int b) {
    return (int)b < (int)a ? b : a;
  }
  static __device__ __forceinline__ unsigned int u(unsigned int a, unsigned int b) { return b < a ? b : a; }
};
struct OpMax {
  static __device__ __forceinline__ float f(float a, float b) { return a < b ? b : a; }
  static __device__ __forceinline__ double d(double a, double b) { return a < b ? b : a; }
  static __device__ __forceinline__ unsigned int i(unsigned int a, unsigned int b) {
    return (int)a < (int)b ? b : a;
  }
  static __device__ __forceinline__ unsigned int u(unsigned int a, unsigned int b) { return a < b ? b : a; }
};

// ---- per-dtype: fold one 32-bit word of every input ------------------------
template <int DT> struct Dtype;

template <> struct Dtype<PCCL_F32> {
  static constexpr int kElemBytes = 4;
  typedef unsigned int elem_t;
  typedef u32x4_a4 pack_unaligned;
  static __device__ __forceinline__ void wave_init() {}
  template <class Op, int N> static __device__ __forceinline__ unsigned int word(const unsigned int (&w)[N]) {
    float acc = as_f32(w[0]);
#pragma unroll
    for (int k = 1; k < N; ++k) acc = Op::f(acc, as_f32(w[k]));
    return as_u32(acc);
  }
  template <class Op, int N> static __device__ __forceinline__ elem_t elem(const elem_t (&e)[N]) {
    return word<Op, N>(e);
  }
};

template <> struct Dtype<PCCL_I32> {
  static constexpr int kElemBytes = 4;
  typedef unsigned int elem_t;
  typedef u32x4_a4 pack_unaligned;
  static __device__ __forceinline__ void wave_init() {}
  template <class Op, int N> static __device__ __forceinline__ unsigned int word(const unsigned int (&w)[N]) {
    unsigned int acc = w[0];
#pragma unroll
    for (int k = 1; k < N; ++k) acc = Op::i(acc, w[k]);
    return acc;
  }
  template <class Op, int N> static __device__ __forceinline__ elem_t elem(const elem_t (&e)[N]) {
    return word<Op, N>(e);
  }
};

template <> struct Dtype<PCCL_U32> {
  static constexpr int kElemBytes = 4;
  typedef unsigned int elem_t;
  typedef u32x4_a4 pack_unaligned;
  static __device__ __forceinline__ void wave_init() {}
  template <class Op, int N> static __device__ __forceinline__ unsigned int word(const unsigned int (&w)[N]) {
    unsigned int acc = w[0];
#pragma unroll
    for (int k = 1; k < N; ++k) acc = Op::u(acc, w[k]);
    return acc;
  }
  template <class Op, int N> static __device__ __forceinline__ elem_t elem(const elem_t (&e)[N]) {
    return word<Op, N>(e);
  }
};

// binary64: an element spans two words, so the fold works on word pairs (fold_pack below)
template <> struct Dtype<PCCL_F64> {
  static constexpr int kElemBytes = 8;
  typedef unsigned long long elem_t;
  typedef u32x4_a8 pack_unaligned;
  static __device__ __forceinline__ void wave_init() {}
  template <class Op, int N> static __device__ __forceinline__ elem_t elem(const elem_t (&e)[N]) {
    double acc = __builtin_bit_cast(double, e[0]);
#pragma unroll
    for (int k = 1; k < N; ++k) acc = Op::d(acc, __builtin_bit_cast(double, e[k]));
    return __builtin_bit_cast(elem_t, acc);
  }
};

template <> struct Dtype<PCCL_BF16> {
  static constexpr int kElemBytes = 2;
  typedef unsigned short elem_t;
  typedef u32x4_a2 pack_unaligned;
  static __device__ __forceinline__ void wave_init() {}
  // two bf16 per word: widen by shifting into the top half of a binary32,
  // fold both halves in float, round once (v_cvt_pk_bf16_f32: nearest even)
  template <class Op, int N> static __device__ __forceinline__ unsigned int word(const unsigned int (&w)[N]) {
    float lo = as_f32(w[0] << 16), hi = as_f32(w[0] & 0xffff0000u);
#pragma unroll
    for (int k = 1; k < N; ++k) {
      lo = Op::f(lo, as_f32(w[k] << 16));
      hi = Op::f(hi, as_f32(w[k] & 0xffff0000u));
    }
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, bf16x2));
  }
  template <class Op, int N> static __device__ __forceinline__ elem_t elem(const elem_t (&e)[N]) {
    float acc = as_f32((unsigned int)e[0] << 16);
#pragma unroll
    for (int k = 1; k < N; ++k) acc = Op::f(acc, as_f32((unsigned int)e[k] << 16));
    return __builtin_bit_cast(unsigned short, (__bf16)acc);
  }
};

template <> struct Dtype<PCCL_F16> {
  static constexpr int kElemBytes = 2;
  typedef unsigned short elem_t;
  typedef u32x4_a2 pack_unaligned;
  static __device__ __forceinline__ void wave_init() {}
  template <class Op, int N> static __device__ __forceinline__ unsigned int word(const unsigned int (&w)[N]) {
    f32x2 acc = __builtin_convertvector(__builtin_bit_cast(f16x2, w[0]), f32x2);
#pragma unroll
    for (int k = 1; k < N; ++k) {
      f32x2 x = __builtin_convertvector(__builtin_bit_cast(f16x2, w[k]), f32x2);
      acc.x = Op::f(acc.x, x.x);
      acc.y = Op::f(acc.y, x.y);
    }
    float lo = acc.x, hi = acc.y;
    rounded_to_f32(lo);
    rounded_to_f32(hi);
    acc.x = lo;
    acc.y = hi;
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(acc, f16x2));
  }
  template <class Op, int N> static __device__ __forceinline__ elem_t elem(const elem_t (&e)[N]) {
    float acc = (float)__builtin_bit_cast(_Float16, e[0]);
#pragma unroll
    for (int k = 1; k < N; ++k) acc = Op::f(acc, (float)__builtin_bit_cast(_Float16, e[k]));
    rounded_to_f32(acc);
    return __builtin_bit_cast(unsigned short, (_Float16)acc);
  }
  // The fold's last step must round to binary32 before the result is narrowed.  Left alone,
  // the compiler folds "multiply a float by a widened half, narrow to half" into one
  // v_fma_mixlo_f16, which rounds the exact product once; where the binary32 product lies
  // exactly between two binary16 values that is one unit away from rounding twice (seen on
  // 1 of ~10^4 head / tail elements of an 8-input product).  The empty asm makes the value
  // opaque to that pattern and costs no instruction.
  static __device__ __forceinline__ void rounded_to_f32(float &x) { asm volatile("" : "+v"(x)); }
};

// 8-bit floats (OCP E4M3FN and E5M2), four per word.  Widening is the hardware's exact
// v_cvt_f32_fp8 / v_cvt_f32_bf8; narrowing is v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32 (round to
// nearest even) with the wave's FP16_OVFL mode bit set, under which a finite value beyond the
// largest finite one saturates to it instead of becoming NaN / infinity, NaN stays NaN and a
// true infinity stays infinite (E5M2) or becomes NaN (E4M3FN, which has no infinity; no fold
// of E4M3FN operands can produce one).  Checked against clamp-then-convert over all 2^32
// binary32 patterns.  wave_init() must run once per wave before the first narrowing.
template <bool E5M2> struct F8Fmt {
  static __device__ __forceinline__ void wave_init() {
    // MODE register (hwreg 1), bit 23 = FP16_OVFL; the clobber keeps loads (and so every
    // conversion of loaded data) behind the mode change
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 1\n\ts_nop 1" ::: "memory");
  }
  static __device__ __forceinline__ float up(unsigned int w, int byte) {
    if constexpr (E5M2) {
      switch (byte) {
        case 0: return __builtin_amdgcn_cvt_f32_bf8(w, 0);
        case 1: return __builtin_amdgcn_cvt_f32_bf8(w, 1);
        case 2: return __builtin_amdgcn_cvt_f32_bf8(w, 2);
        default: return __builtin_amdgcn_cvt_f32_bf8(w, 3);
      }
    } else {
      switch (byte) {
        case 0: return __builtin_amdgcn_cvt_f32_fp8(w, 0);
        case 1: return __builtin_amdgcn_cvt_f32_fp8(w, 1);
        case 2: return __builtin_amdgcn_cvt_f32_fp8(w, 2);
        default: return __builtin_amdgcn_cvt_f32_fp8(w, 3);
      }
    }
  }
  // two at a time: bytes 0,1 (hi = false) or 2,3 (hi = true) of w
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  template <bool HI> static __device__ __forceinline__ f32x2 up2(unsigned int w) {
    if constexpr (E5M2) return __builtin_amdgcn_cvt_pk_f32_bf8((int)w, HI);
    else return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, HI);
  }
  static __device__ __forceinline__ unsigned int down4(float a, float b, float c, float d) {
    int p = 0;
    if constexpr (E5M2) {
      p = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, p, false);
      p = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, p, true);
    } else {
      p = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, p, false);
      p = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, p, true);
    }
    return (unsigned int)p;
  }
};

template <bool E5M2> struct DtypeF8 {
  typedef F8Fmt<E5M2> F;
  static constexpr int kElemBytes = 1;
  typedef unsigned char elem_t;
  typedef u32x4_a1 pack_unaligned;
  static __device__ __forceinline__ void wave_init() { F::wave_init(); }
  template <class Op, int N> static __device__ __forceinline__ unsigned int word(const unsigned int (&w)[N]) {
    typename F::f32x2 lo = F::template up2<false>(w[0]), hi = F::template up2<true>(w[0]);
    float a = lo.x, b = lo.y, c = hi.x, d = hi.y;
#pragma unroll
    for (int k = 1; k < N; ++k) {
      lo = F::template up2<false>(w[k]);
      hi = F::template up2<true>(w[k]);
      a = Op::f(a, lo.x);
      b = Op::f(b, lo.y);
      c = Op::f(c, hi.x);
      d = Op::f(d, hi.y);
    }
    return F::down4(a, b, c, d);
  }
  template <class Op, int N> static __device__ __forceinline__ elem_t elem(const elem_t (&e)[N]) {
    float acc = F::up((unsigned int)e[0], 0);
#pragma unroll
    for (int k = 1; k < N; ++k) acc = Op::f(acc, F::up((unsigned int)e[k], 0));
    return (elem_t)(F::down4(acc, 0.0f, 0.0f, 0.0f) & 0xffu);
  }
};
template <> struct Dtype<PCCL_F8E4M3> : DtypeF8<false> {};
template <> struct Dtype<PCCL_F8E5M2> : DtypeF8<true> {};

// ---- pack load / store -------------------------------------------------------
// A pack is addressed as (base, off): `base` is the same for every lane of the wavefront
// (it sits in scalar registers), `off` is the lane's byte offset, below 4 GiB.
// ALIGNED: every stream is 16-byte aligned.  Otherwise only output 0 is (the
// host peels a head so that it is) and the others are element-aligned.
//
// Memory policy of an access:
//   kMemCached    ordinary cached access;
//   kMemStream    non-temporal hint (operands larger than the Infinity Cache);
//   kMemCoherent  device-coherent access (sc1): loads read past, and stores write
//                 through, this XCD's L2, which is not coherent with the L2s of the
//                 other seven XCDs.  Used where workgroups on different XCDs hand
//                 data to each other inside one kernel, so that no L2-wide
//                 write-back / invalidate is needed at every hand-over, and for the
//                 stores of large reductions.  The compiler offers sc1 on global
//                 accesses only for atomics of at most 8 bytes, so these go through
//                 the buffer instructions, whose cache-policy operand it exposes
//                 (buffer_load_dwordx4 ... nt sc1 / buffer_store_dwordx4 ... sc1); wait counts and
//                 instruction hazards stay the compiler's business.
constexpr int kMemCached = 0, kMemStream = 1, kMemCoherent = 2;

// cache-policy operand of the buffer builtins on this target: 1 = sc0, 2 = nt, 16 = sc1
constexpr int kCachePolicySc1 = 16;
// Coherent loads also carry the non-temporal hint: what a part reads it reads once (14 ops of
// 32 MiB through the queue: 258 -> 235 us; the 4096-op schedule is unchanged).
constexpr int kCachePolicyNtSc1 = 2 | 16;

// Buffer resource over the whole address space above `base`: no stride, no bounds
// clamp below 4 GiB, raw 32-bit data (word 3 as for every gfx9-family part).
// `base` is wave-uniform by contract; reading it from the first lane tells the compiler so
// where it cannot prove it (the descriptor must sit in scalar registers, and for a base
// it takes to be lane-varying it would build a loop over the distinct values).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t whole_buffer(const void *base) {
  const unsigned long long b = (unsigned long long)base;
  // readfirstlane returns int: go through unsigned int, or a low word with its top bit set
  // would sign-extend into the high word
  const unsigned int lo = (unsigned int)__builtin_amdgcn_readfirstlane((int)(unsigned int)b);
  const unsigned int hi = (unsigned int)__builtin_amdgcn_readfirstlane((int)(unsigned int)(b >> 32));
  const unsigned long long uniform = (unsigned long long)lo | ((unsigned long long)hi << 32);
  return __builtin_amdgcn_make_buffer_rsrc((void *)uniform, 0, (int)0xffffffffu, 0x00020000);
}

template <class D, bool ALIGNED, int MEM>
__device__ __forceinline__ u32x4 load_pack(const char *base, unsigned int off) {
  if constexpr (MEM == kMemCoherent) {
    return __builtin_amdgcn_raw_buffer_load_b128(whole_buffer(base), (int)off, 0, kCachePolicyNtSc1);
  } else if constexpr (ALIGNED) {
    if constexpr (MEM == kMemStream) return __builtin_nontemporal_load((const u32x4 *)(base + off));
    else return *(const u32x4 *)(base + off);
  } else {
    typedef typename D::pack_unaligned P;
    if constexpr (MEM == kMemStream) return __builtin_nontemporal_load((const P *)(base + off));
    else return *(const P *)(base + off);
  }
}

template <class D, bool ALIGNED, int MEM>
__device__ __forceinline__ void store_pack(char *base, unsigned int off, u32x4 v) {
  if constexpr (MEM == kMemCoherent) {
    __builtin_amdgcn_raw_buffer_store_b128(v, whole_buffer(base), (int)off, 0, kCachePolicySc1);
  } else if constexpr (ALIGNED) {
    if constexpr (MEM == kMemStream) __builtin_nontemporal_store(v, (u32x4 *)(base + off));
    else *(u32x4 *)(base + off) = v;
  } else {
    typedef typename D::pack_unaligned P;
    if constexpr (MEM == kMemStream) __builtin_nontemporal_store(v, (P *)(base + off));
    else *(P *)(base + off) = v;
  }
}

// Waits until every coherent store issued by this wavefront has reached the
// point of coherence (needed before another workgroup is told the data exists).
__device__ __forceinline__ void settle_stores() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); }

template <class E, int MEM>
__device__ __forceinline__ E load_elem(const E *p) {
  if constexpr (MEM == kMemCoherent) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else return *p;
}

template <class E, int MEM>
__device__ __forceinline__ void store_elem(E *p, E v) {
  if constexpr (MEM == kMemCoherent) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else *p = v;
}

template <class D, class Op, int NIN>
__device__ __forceinline__ u32x4 fold_pack(const u32x4 (&v)[NIN]) {
  if constexpr (NIN == 1) {
    return v[0];  // COPY: bytes unchanged
  } else {
    u32x4 r;
    if constexpr (D::kElemBytes == 8) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        unsigned long long e[NIN];
#pragma unroll
        for (int k = 0; k < NIN; ++k) e[k] = (unsigned long long)v[k][2 * j] | ((unsigned long long)v[k][2 * j + 1] << 32);
        const unsigned long long x = D::template elem<Op, NIN>(e);
        r[2 * j] = (unsigned int)x;
        r[2 * j + 1] = (unsigned int)(x >> 32);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        unsigned int w[NIN];
#pragma unroll
        for (int k = 0; k < NIN; ++k) w[k] = v[k][j];
        r[j] = D::template word<Op, NIN>(w);
      }
    }
    return r;
  }
}

// Operands of one reduce-copy (or of one part of it), as the kernels see them.
struct RcOperands {
  const char *in[PCCL_MAX_INPUTS];
  char *out[PCCL_MAX_OUTPUTS];
  int n_out;
};

// Body: packs [0, n_packs) of every stream, stream pointers already at the
// first pack.  Workgroup `wg` of `n_wg` takes chunks wg, wg+n_wg, ... of
// kBlock*UNROLL packs; inside a chunk lane t takes packs t, t+kBlock, ... so
// every load and store instruction of a wavefront covers 1 KiB contiguously.
//
// LD / ST are the memory policies of loads / stores.  Measured on MI355X with
// buffers far larger than the 256 MB Infinity Cache: reductions want both
// streaming, a plain copy wants only the stores; cache-resident sizes want neither.
template <class D, class Op, int NIN, int UNROLL, bool ALIGNED, int LD, int ST>
__device__ __forceinline__ void body_packs(const RcOperands &a, long n_packs, long wg, long n_wg) {
  constexpr long kChunk = (long)kBlock * UNROLL;
  for (long base = wg * kChunk; base < n_packs; base += n_wg * kChunk) {
    const size_t chunk = (size_t)base * 16;  // byte offset of the chunk: the same for every lane
    if (base + kChunk <= n_packs) {
      u32x4 v[UNROLL][NIN];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u)
#pragma unroll
        for (int k = 0; k < NIN; ++k)
          v[u][k] = load_pack<D, ALIGNED, LD>(a.in[k] + chunk, (threadIdx.x + (unsigned)u * kBlock) * 16u);
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const u32x4 r = fold_pack<D, Op, NIN>(v[u]);
        const unsigned int off = (threadIdx.x + (unsigned)u * kBlock) * 16u;
        store_pack<D, true, ST>(a.out[0] + chunk, off, r);
#pragma unroll
        for (int j = 1; j < PCCL_MAX_OUTPUTS; ++j)
          if (j < a.n_out) store_pack<D, ALIGNED, ST>(a.out[j] + chunk, off, r);
      }
    } else if constexpr (D::kElemBytes == 1 && NIN > 1) {
      // last, partial chunk, 8-bit floats: pack by pack (the batched form below costs them a
      // wavefront per SIMD in registers)
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const unsigned int off = (threadIdx.x + (unsigned)u * kBlock) * 16u;
        if (base + threadIdx.x + (long)u * kBlock < n_packs) {
          u32x4 v[NIN];
#pragma unroll
          for (int k = 0; k < NIN; ++k) v[k] = load_pack<D, ALIGNED, LD>(a.in[k] + chunk, off);
          const u32x4 r = fold_pack<D, Op, NIN>(v);
          store_pack<D, true, ST>(a.out[0] + chunk, off, r);
#pragma unroll
          for (int j = 1; j < PCCL_MAX_OUTPUTS; ++j)
            if (j < a.n_out) store_pack<D, ALIGNED, ST>(a.out[j] + chunk, off, r);
        }
      }
    } else {  // last, partial chunk: same shape; a lane without a pack u re-reads the chunk's
      // last pack (so that all loads still go out together) and stores nothing for it
      const unsigned int last = (unsigned int)(n_packs - base - 1);
      u32x4 v[UNROLL][NIN];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const unsigned int p = threadIdx.x + (unsigned)u * kBlock;
#pragma unroll
        for (int k = 0; k < NIN; ++k) v[u][k] = load_pack<D, ALIGNED, LD>(a.in[k] + chunk, (p < last ? p : last) * 16u);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const unsigned int p = threadIdx.x + (unsigned)u * kBlock;
        if (p <= last) {
          const u32x4 r = fold_pack<D, Op, NIN>(v[u]);
          store_pack<D, true, ST>(a.out[0] + chunk, p * 16u, r);
#pragma unroll
          for (int j = 1; j < PCCL_MAX_OUTPUTS; ++j)
            if (j < a.n_out) store_pack<D, ALIGNED, ST>(a.out[j] + chunk, p * 16u, r);
        }
      }
    }
  }
}

// Edge elements, one per lane of a single wavefront: elements [0, head) and
// [tail_begin, count) of the ORIGINAL (un-advanced) streams.
template <class D, class Op, int NIN, int MEM = kMemCached>
__device__ __forceinline__ void edge_elems(const RcOperands &a, long head, long tail_begin,
                                           long count, int lane) {
  typedef typename D::elem_t E;
  const long n_edge = head + (count - tail_begin);
  for (long e = lane; e < n_edge; e += kWave) {
    const long i = e < head ? e : tail_begin + (e - head);
    E x[NIN];
#pragma unroll
    for (int k = 0; k < NIN; ++k) x[k] = load_elem<E, MEM>((const E *)a.in[k] + i);
    E r;
    if constexpr (NIN == 1) r = x[0];
    else r = D::template elem<Op, NIN>(x);
#pragma unroll
    for (int j = 0; j < PCCL_MAX_OUTPUTS; ++j)
      if (j < a.n_out) store_elem<E, MEM>((E *)a.out[j] + i, r);
  }
}

}  // namespace pccl_dev
