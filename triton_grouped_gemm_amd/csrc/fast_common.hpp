// Building blocks shared by the tuned gfx950 GEMM kernels: direct-to-LDS slab copies, their buffer
// descriptors, the vmcnt bookkeeping and the swizzled slab geometry.
#pragma once
#include "common.hpp"
#include "sched.hpp"

namespace tgg {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(3))) i16x4_t* lds_i16x4_ptr_t;

// s_waitcnt vmcnt(n) only (gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]).
template <int N> TGG_DEV void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// All of this wave's vector-memory traffic and all of its LDS reads have completed.
TGG_DEV void wait_vmcnt0_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(7 << 4); }

// One wave-wide 16-byte-per-lane copy global -> LDS.  The LDS destination is m0 + lane * 16, the
// global source is the descriptor base + voff (bounds-checked: out-of-range lanes write zeros).
// Written as inline assembly on purpose: the compiler does not model the copy, so it cannot
// serialise the software pipeline with conservative waits; completion is tracked by hand with
// wait_vmcnt<>() and the workgroup barrier.  s_nop 0: a copy to LDS that follows a scalar write of m0 needs one wait
// state in between on this hardware generation (the compiler inserts it for its own such copies and does not look
// inside this statement).
TGG_DEV void copy_b128_to_lds(i32x4_t rsrc, uint32_t lds_addr, int voff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" : : "s"(lds_addr), "v"(voff), "s"(rsrc) : "memory", "m0");
}

// Output store of the tuned kernels; dst is global memory.  nt = non-temporal: the output is written once and
// not read again by the kernel, and with the nt bit the lines do not compete with the operand panels that the
// other CUs of the XCD keep re-reading from L2 (+4 % on a store-heavy shape, K = 768).  The bit is set through
// the instruction text: the compiler's non-temporal store builtin did not have that effect here.
TGG_DEV void store_c(i32x4_t* dst, i32x4_t v, int nt) {
  // s_nop 1: a vector instruction that overwrites the data registers of a 16-byte store within two wait states
  // corrupts what is stored, and the compiler, which considers them free after this statement, does not look inside it.
  if (nt) asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" : : "v"(dst), "v"(v) : "memory");
  else *(__attribute__((address_space(1))) i32x4_t*)(uint64_t)dst = v;
}

// Pins a wave-uniform 64-bit value to a scalar register pair.
TGG_DEV uint64_t uniform64(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

// Raw buffer descriptor over [base, base + bytes), bytes clamped to [0, 2^31).
TGG_DEV i32x4_t make_rsrc(uint64_t base, int64_t bytes) {
  bytes = bytes < 0 ? 0 : (bytes > 0x7fffffff ? 0x7fffffff : bytes);
  i32x4_t r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)base);
  r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(base >> 32) & 0xffff);  // stride 0, no swizzle
  r[2] = __builtin_amdgcn_readfirstlane((int)bytes);
  r[3] = 0x00020000;  // 32-bit data format
  return r;
}

// The same with a 32-bit length (negative = nothing left).
TGG_DEV i32x4_t make_rsrc32(uint64_t base, int bytes) {
  i32x4_t r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)base);
  r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(base >> 32) & 0xffff);  // stride 0, no swizzle
  r[2] = __builtin_amdgcn_readfirstlane(bytes < 0 ? 0 : bytes);
  r[3] = 0x00020000;  // 32-bit data format
  return r;
}

constexpr int kFastMaxGroups = 512;
constexpr int kSlabRowBytes = 128;  // a slab holds 128 bytes of every K-contiguous row (64 bf16 / 128 fp8 values)

// Geometry of one operand's slab in LDS and of the copies that fill it.
//   KMAJOR: ROWS rows of 128 bytes (64 K values each).  A copy instruction covers 8 rows; the
//           16-byte chunk c of row r sits at slot c ^ ((r / 2) % 8).
//   !KMAJOR: 64 token rows of ROWS*2 bytes.  A copy instruction covers 1024 / (ROWS*2) token rows;
//           chunk c of token row k sits at slot c ^ ((k % 4) * 4) ^ ((k / 8 % 2) * 2): the transposing fragment
//           read of a wave touches token rows 8 g + e (g = 0..3, e = 0..3) at the same columns, and this spreads
//           them over all banks.
template <int ROWS, bool KMAJOR> struct Operand {
  static constexpr int SLAB_BYTES = ROWS * kSlabRowBytes;
  static constexpr int NI = SLAB_BYTES / 1024;                 // copy instructions per slab
  static constexpr int ROW_BYTES = KMAJOR ? kSlabRowBytes : ROWS * 2;  // bytes of one LDS row (token rows: 16-bit)
  static constexpr int CPR = ROW_BYTES / 16;                   // 16-byte chunks per LDS row
  static constexpr int RPI = 1024 / ROW_BYTES;                 // LDS rows per copy instruction
  static constexpr int NPAT = KMAJOR ? 2 : (RPI >= 16 ? 1 : 16 / RPI);  // swizzle patterns over instructions

  // byte offset (from the slab's first byte in global memory) fetched by `lane` of a copy
  // instruction with swizzle pattern `pat`; ld = bytes between consecutive global rows.
  static TGG_DEV int lane_voff(int lane, int pat, int ld) {
    const int r_local = lane / CPR, slot = lane % CPR;
    const int r = pat * RPI + r_local;  // row index modulo the swizzle period
    const int sw = KMAJOR ? (r / 2) % 8 : ((r % 4) * 4) ^ ((r / 8 % 2) * 2);
    return r_local * ld + ((slot ^ sw) << 4);
  }
  // K-contiguous rows only: which 16-byte chunk of its row (0..7) that lane fetches
  static TGG_DEV int lane_chunk(int lane, int pat) {
    const int r = pat * RPI + lane / CPR;
    return (lane % CPR) ^ ((r / 2) % 8);
  }
};

// A source offset no descriptor of the tuned kernels reaches (their operand windows stay below 1 GiB):
// a lane given this offset fetches nothing and writes zeros.
constexpr int kNoFetch = 0x40000000;

}  // namespace tgg
