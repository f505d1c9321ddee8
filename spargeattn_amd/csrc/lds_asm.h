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
// Reads that nothing is overlapped with carry their wait in the SAME asm statement: the outputs become visible to the
// compiler only once they are valid, so no copy, spill or live-range split can ever observe a register in flight.
// a <- addr0 + O0, b <- addr0 + O1, c <- addr1 + O0, d <- addr1 + O1.
template <int O0, int O1>
__device__ __forceinline__ void lds_read_4x128_wait(v4i &a, v4i &b, v4i &c, v4i &d, uint32_t addr0, uint32_t addr1) {
  asm volatile("ds_read_b128 %0, %4 offset:%6\n\tds_read_b128 %1, %4 offset:%7\n\t"
               "ds_read_b128 %2, %5 offset:%6\n\tds_read_b128 %3, %5 offset:%7\n\ts_waitcnt lgkmcnt(0)"
               : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d)
               : "v"(addr0), "v"(addr1), "n"(O0), "n"(O1)
               : "memory");
}
// a, b, c, d <- addr0 + O0 .. O3; e, f, g, h <- addr1 + O0 .. O3
template <int O0, int O1, int O2, int O3>
__device__ __forceinline__ void lds_read_8x128_wait(v4i &a, v4i &b, v4i &c, v4i &d, v4i &e, v4i &f, v4i &g, v4i &h,
                                                    uint32_t addr0, uint32_t addr1) {
  asm volatile("ds_read_b128 %0, %8 offset:%10\n\tds_read_b128 %1, %8 offset:%11\n\t"
               "ds_read_b128 %2, %8 offset:%12\n\tds_read_b128 %3, %8 offset:%13\n\t"
               "ds_read_b128 %4, %9 offset:%10\n\tds_read_b128 %5, %9 offset:%11\n\t"
               "ds_read_b128 %6, %9 offset:%12\n\tds_read_b128 %7, %9 offset:%13\n\ts_waitcnt lgkmcnt(0)"
               : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d), "=&v"(e), "=&v"(f), "=&v"(g), "=&v"(h)
               : "v"(addr0), "v"(addr1), "n"(O0), "n"(O1), "n"(O2), "n"(O3)
               : "memory");
}
// a <- addr0 + O0, b <- addr1 + O1
template <int O0, int O1>
__device__ __forceinline__ void lds_read_2x128_wait(v4i &a, v4i &b, uint32_t addr0, uint32_t addr1) {
  asm volatile("ds_read_b128 %0, %2 offset:%4\n\tds_read_b128 %1, %3 offset:%5\n\ts_waitcnt lgkmcnt(0)"
               : "=&v"(a), "=&v"(b)
               : "v"(addr0), "v"(addr1), "n"(O0), "n"(O1)
               : "memory");
}
// The split forms below (reads here, wait later) remain for the groups whose latency runs under matrix instructions.
// Between such a read and its wait the destination registers are "written" as far as the compiler knows: the kernels
// that use them are built with a check that nothing is spilled, and the build records the compiler version the
// generated code was inspected with.
// wait for all outstanding LDS reads; the operands tie the wait to the registers it makes valid
__device__ __forceinline__ void lds_wait4(v4i &a, v4i &b, v4i &c, v4i &d) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
__device__ __forceinline__ void lds_wait2(v4i &a, v4i &b) { asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b)); }

}  // namespace spg
