// Shared device helpers for the gfx950 (CDNA4) Pairformer pair-stack kernels.
//
// MFMA convention used by every kernel in this directory ("mma32"):
//   acc[32 x 32] += A[32 x 16] * B[16 x 32]
//   lane l supplies row    m = l % 32 of A, K-slots 8*(l/32) .. 8*(l/32)+7
//   lane l supplies column n = l % 32 of B, the same K-slots
//   lane l receives column n = l % 32 of acc; register r holds row
//        8*(r/4) + 4*(l/32) + (r%4)
// An operand "fragment" is therefore 8 consecutive K elements per lane, for
// bf16 (one v_mfma_f32_32x32x16_bf16) and for fp32 (eight
// v_mfma_f32_32x32x2_f32, slot t of both operands per instruction).  Because
// both operands use the same slot numbering, which physical K index a slot
// stands for is the kernel's choice.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ptx {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;   // IEEE half: the stand-alone LayerNorm only
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kWave = 64;

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> { typedef bf16x8 type; };
template <> struct Vec8<float> { typedef f32x8 type; };
template <typename T> struct Vec4;
template <> struct Vec4<bf16_t> { typedef bf16x4 type; };
template <> struct Vec4<float> { typedef f32x4 type; };

__device__ __forceinline__ f32x8 to_f32(bf16x8 v) { return __builtin_convertvector(v, f32x8); }
__device__ __forceinline__ f32x8 to_f32(f32x8 v) { return v; }
__device__ __forceinline__ f32x4 to_f32(bf16x4 v) { return __builtin_convertvector(v, f32x4); }
__device__ __forceinline__ f32x4 to_f32(f32x4 v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(float v) { return v; }

template <typename T> __device__ __forceinline__ typename Vec8<T>::type from_f32(f32x8 v);
template <> __device__ __forceinline__ bf16x8 from_f32<bf16_t>(f32x8 v) { return __builtin_convertvector(v, bf16x8); }
template <> __device__ __forceinline__ f32x8 from_f32<float>(f32x8 v) { return v; }
template <typename T> __device__ __forceinline__ typename Vec4<T>::type from_f32(f32x4 v);
template <> __device__ __forceinline__ bf16x4 from_f32<bf16_t>(f32x4 v) { return __builtin_convertvector(v, bf16x4); }
template <> __device__ __forceinline__ f32x4 from_f32<float>(f32x4 v) { return v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }
template <> __device__ __forceinline__ f16_t from_f32<f16_t>(float v) { return (f16_t)v; }
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }

// acc += A * B for one 16-deep K step (see the convention above).
__device__ __forceinline__ void mma32(f32x16& acc, bf16x8 a, bf16x8 b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}
__device__ __forceinline__ void mma32(f32x16& acc, f32x8 a, f32x8 b) {
#pragma unroll
  for (int t = 0; t < 8; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], acc, 0, 0, 0);
}

// Row of acc held by register r of a lane in half-wave g (= lane / 32).
__device__ __forceinline__ int acc_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

// Value of the lane 32 places away (the other half-wave).
__device__ __forceinline__ float swap32(float v) { return __shfl_xor(v, 32, 64); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
// sigmoid(x) = 1 / (1 + 2^(-x*log2 e)); |rel err| ~ 1e-7, saturates cleanly at +-inf.
__device__ __forceinline__ float sigmoidf_fast(float x) {
  return fast_rcp(1.0f + fast_exp2(-1.4426950408889634f * x));
}

// 16-byte (8 x bf16) or 32-byte (8 x fp32) global accesses.
template <typename T>
__device__ __forceinline__ typename Vec8<T>::type load8(const T* p) {
  return *reinterpret_cast<const typename Vec8<T>::type*>(p);
}
template <typename T>
__device__ __forceinline__ void store8(T* p, typename Vec8<T>::type v) {
  *reinterpret_cast<typename Vec8<T>::type*>(p) = v;
}

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

// Direct-to-LDS load: every lane moves 16 bytes from its own global address to LDS address
// lds_base + 16 * lane (M0 carries the base).  Issued as inline asm on purpose: for
// direct-to-LDS loads it knows about, the compiler waits for ALL of them (vmcnt(0)) before
// any later LDS read, which would serialise a ring whose loads run stages ahead.  The
// waits are placed by hand in ring_barrier() instead.
// (M0 is a reserved register, which the compiler warns about in a clobber list; the
// clobber is what tells it to re-initialise M0 before its own next use.)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void load_to_lds16(const void* gptr, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gptr), "s"(lds_base)
               : "m0");
}
// The same with the address split into a wave-uniform 64-bit base (scalar registers), a
// 32-bit byte offset per lane and an immediate: no vector ALU work per load.  The immediate
// is added to the LDS address as well as to the global one.
template <int IMM>
__device__ __forceinline__ void load_to_lds16_s(uint64_t sbase, uint32_t voff, uint32_t lds_base) {
  static_assert(IMM >= 0 && IMM < 4096, "13-bit signed immediate offset");
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
               :
               : "v"(voff), "s"(sbase), "s"(lds_base), "n"(IMM)
               : "m0");
}
// A 64-bit value that is the same in all lanes, moved to scalar registers.
__device__ __forceinline__ uint64_t uniform64(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}
#pragma clang diagnostic pop
// LDS byte address of p, which must be the same for all lanes (it goes to a scalar register)
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p);
}

// Workgroup barrier for the stage ring: wait until all but the N youngest direct-to-LDS
// loads of this wave have landed and all its LDS reads have returned, then s_barrier.
// The memory clobbers keep the compiler from moving LDS accesses across the barrier.
template <int N> __device__ __forceinline__ void ring_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// Position of a logical pair-tensor row p = outer * n_inner + inner in a tensor
// whose (outer, inner) axes have arbitrary element strides.  The ending-node
// attention and the incoming triangle product read z[inner, outer] this way,
// so no transposed copy of the pair tensor is ever made.
struct RowMap {
  int64_t stride_outer;
  int64_t stride_inner;
  int n_inner;
  // p < 2^31 (the API bounds n and the row counts), so 32-bit division suffices
  __device__ __forceinline__ int64_t operator()(int64_t p) const {
    const uint32_t pp = (uint32_t)p;
    const uint32_t o = pp / (uint32_t)n_inner;
    const uint32_t i = pp - o * (uint32_t)n_inner;
    return (int64_t)o * stride_outer + (int64_t)i * stride_inner;
  }
};

// ---------------------------------------------------------------------------
// Operand layout of the triangle-multiplication contraction (written by the
// projection kernel, read by the contraction): per channel, rows in blocks of 32
// and K in steps of 16; one (row block, K step) fragment is stored in MFMA
// operand order, 64 lanes x 8 elements = 512 contiguous elements: lane
// 32*g + r holds K = 16*ks + 8*g .. +7 of row 32*rb + r.  A channel has
// ceil(n/32) row blocks (rows beyond n are never written) and k_pitch/16 K steps
// (K between n and k_pitch is written as zeros: the contraction runs over it).
// ---------------------------------------------------------------------------
constexpr int kFragElems = 512;

__host__ __device__ __forceinline__ int64_t trimul_frag_offset(int c, int rb, int ks, int n_rb,
                                                               int n_ks) {
  return (((int64_t)c * n_rb + rb) * n_ks + ks) * kFragElems;
}

// ---------------------------------------------------------------------------
// Operand layouts of the triangle-attention core (written by the projection
// kernel, read by the attention kernel).  Keys are grouped in tiles of 64; one
// operand tile is stored in MFMA fragment order, 4 fragments x 64 lanes x 8
// elements, so that every fragment load of the attention kernel is one fully
// contiguous 1 KB (bf16) read.  Within a key tile, key jj = 32*g + 16*u + r:
//   K   fragment (u, kk): lane 32*gl + m holds d = 16*kk + 8*gl .. +7 of the key
//       whose MFMA row is m = 8*(r>>2) + 4*g + (r&3)
//   V^T fragment (u, s):  lane 32*g + d holds keys 32*g + 16*u + 8*s .. +7 of channel d
//   bias fragment (u, c): lane 32*g + q holds keys 32*g + 16*u + 8*c .. +7 of query q
//       (queries in blocks of 32)
// q, the gate and the output are head-major: [head][i][j][32].
// ---------------------------------------------------------------------------
constexpr int kAttnTileElems = 2048;   // 4 fragments x 64 lanes x 8

__host__ __device__ __forceinline__ int64_t attn_k_offset(int h, int i, int j, int d, int n,
                                                          int key_tiles) {
  const int jj = j & 63, g = jj >> 5, u = (jj >> 4) & 1, r = jj & 15;
  const int m = 8 * (r >> 2) + 4 * g + (r & 3);
  const int c8 = d >> 3, kk = c8 >> 1, gl = c8 & 1;
  return ((((int64_t)h * n + i) * key_tiles + (j >> 6)) * 4 + (u * 2 + kk)) * 512 +
         (32 * gl + m) * 8 + (d & 7);
}
__host__ __device__ __forceinline__ int64_t attn_v_offset(int h, int i, int j, int d, int n,
                                                          int key_tiles) {
  const int jj = j & 63, g = jj >> 5, u = (jj >> 4) & 1, sg = (jj >> 3) & 1;
  return ((((int64_t)h * n + i) * key_tiles + (j >> 6)) * 4 + (u * 2 + sg)) * 512 +
         (32 * g + d) * 8 + (j & 7);
}
__host__ __device__ __forceinline__ int64_t attn_b_offset(int h, int q, int j, int q_blocks,
                                                          int key_tiles) {
  const int jj = j & 63, g = jj >> 5, u = (jj >> 4) & 1, c = (jj >> 3) & 1;
  return ((((int64_t)h * q_blocks + (q >> 5)) * key_tiles + (j >> 6)) * 4 + (u * 2 + c)) * 512 +
         (32 * g + (q & 31)) * 8 + (j & 7);
}

}  // namespace ptx
