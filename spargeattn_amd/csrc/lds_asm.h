// LDS operand reads and waits through inline asm, shared by the attention kernels whose K/V tiles arrive by
// direct-to-LDS loads (global_load_lds).
#pragma once
#include "common.h"

namespace spg {

typedef int v4i __attribute__((ext_vector_type(4)));

// LDS tile reads are issued through inline asm with explicit waits.  Left to the compiler, every LDS read would be
// ordered after ALL outstanding direct-to-LDS loads of the ring (s_waitcnt vmcnt(0)), which serialises the prefetch
// of block it+2 with the compute of block it.  The ring's own protocol (vmcnt(0) + barrier before a slot is read)
// is what guarantees correctness.
template <int OFF0, int OFF1>
__device__ __forceinline__ void lds_read_2x128(v4i &a, v4i &b, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %2 offset:%3\n\tds_read_b128 %1, %2 offset:%4"
               : "=&v"(a), "=&v"(b)
               : "v"(addr), "n"(OFF0), "n"(OFF1)
               : "memory");
}
// two reads at the same immediate offset from two addresses (the two key chunks of a V^T row)
template <int OFF>
__device__ __forceinline__ void lds_read_pair(v4i &a, v4i &b, uint32_t addr_a, uint32_t addr_b) {
  asm volatile("ds_read_b128 %0, %2 offset:%4\n\tds_read_b128 %1, %3 offset:%4"
               : "=&v"(a), "=&v"(b)
               : "v"(addr_a), "v"(addr_b), "n"(OFF)
               : "memory");
}
// wait for all outstanding LDS reads; the operands tie the wait to the registers it makes valid
__device__ __forceinline__ void lds_wait4(v4i &a, v4i &b, v4i &c, v4i &d) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
__device__ __forceinline__ void lds_wait2(v4i &a, v4i &b) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b)); }

}  // namespace spg
