// LDS reads written as inline assembly, and compile-time loops for their offsets and wait counts.
#pragma once
#include <utility>

#include "common.h"

namespace niti {

#define NITI_LDS(p) ((__attribute__((address_space(3))) void*)(p))
// the same from a 32-bit LDS byte address (no generic pointer, hence no null test in scalar code)
#define NITI_LDS_AT(addr) (reinterpret_cast<__attribute__((address_space(3))) void*>(static_cast<unsigned>(addr)))

// ds_read_b64_tr_b8 as inline assembly.  Before the builtin form the compiler places s_waitcnt vmcnt(0) whenever a
// buffer_load ... lds is in flight (it cannot tell which LDS bytes that load writes), which would make every stage
// wait for the loads it has just issued.  The compiler does not count these reads either: the caller waits with
// lds_settle<N>() - at most N LDS operations issued after the wanted ones still in flight; operations the compiler
// adds in between only make that wait stricter - and passes the results through lds_landed() before using them.
template <int OFF>
__device__ inline v2i lds_read_tr8(unsigned addr) {
  v2i r;
  asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
__device__ inline v4i lds_read_b128(unsigned addr) {
  v4i r;
  asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr));
  return r;
}
template <int OFF>
__device__ inline v4i lds_read_b128_at(unsigned addr) {
  v4i r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
template <int N>
__device__ inline void lds_settle() {
  asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N));
}
__device__ inline v4i lds_landed(v2i lo, v2i hi) {
  asm volatile("" : "+v"(lo), "+v"(hi));
  return v4i{lo[0], lo[1], hi[0], hi[1]};
}
__device__ inline unsigned lds_addr(const void* p) { return static_cast<unsigned>(reinterpret_cast<uintptr_t>(NITI_LDS(p))); }

template <class F, int... I>
__device__ inline void static_for_impl(F& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ inline void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

}  // namespace niti
