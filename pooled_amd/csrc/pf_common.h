// Device helpers shared by the two prefill kernels (gfx950).
#pragma once
#include "pa_internal.h"
#include <hip/hip_fp16.h>
#include <type_traits>

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef __fp16 hh4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));

#define NEG_INF (-__builtin_inff())
#define PF_TN 32                 // positions per step
#ifndef PF_QR
#define PF_QR 16                 // head_dim 256: k-steps of Q kept in registers (any others are parked in LDS)
#endif
#ifndef PF_KD
#define PF_KD 2                  // K (and parked Q) fragments fetched this many k-steps ahead
#endif
#ifndef PF_VD
#define PF_VD 2                  // V^T fragments fetched this many MFMAs ahead
#endif
#define PF_RESCALE_TH 8.0f       // log2 units

static __device__ inline h4 lds_read_tr16(const unsigned char* p) {
  hh4 t = __builtin_amdgcn_ds_read_tr16_b64_v4f16((hh4 __attribute__((address_space(3)))*)p);
  h4 r; __builtin_memcpy(&r, &t, 8); return r;
}

// LDS-direct load of 64 x 16 bytes: lane i's 16 bytes land at LDS byte address lds_addr + 16 i (lds_addr is
// wave-uniform and goes through M0).  Issued as inline assembly on purpose: the compiler then keeps ordinary
// partial lgkmcnt waits for the LDS fragment reads around it (with its own LDS-DMA bookkeeping every LDS wait
// becomes lgkmcnt(0)), and the only wait for these loads is the explicit vmcnt(0) before the end-of-step barrier.
static __device__ inline void pf_gll(const unsigned char* gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(lds_addr), "v"(gptr) : "memory");
}
static __device__ inline uint32_t lds_addr_of(const unsigned char* p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) unsigned char*)p;
}
#define PF_GLL(gptr, lptr) pf_gll((gptr), __builtin_amdgcn_readfirstlane(lds_addr_of(lptr)))
// the same with the address as a wave-uniform base (scalar registers) + a 32-bit per-lane byte offset: the offset is the
// same for every tile, so no 64-bit per-lane addresses are kept or rebuilt
static __device__ inline void pf_gll_s(const unsigned char* sbase, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
#define PF_GLL_S(sbase, voff, lptr) pf_gll_s((sbase), (voff), __builtin_amdgcn_readfirstlane(lds_addr_of(lptr)))
