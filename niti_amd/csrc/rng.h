// Random words drawn inside the kernels (dropout masks, the stochastic rounding of the loss gradient): the
// reference draws them with torch.randint on the device (ti_torch.py:444, ti_loss.py:35 via StoShift), one launch
// each; here they are a function of a small state in device memory, so a kernel that needs them draws them itself.
//
// Generator: Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11).
// State = four uint32 words in device memory: {key0, key1, step, arrivals}.  Word i of stream s in the launch that
// reads `step` = t is output word (i & 3) of philox4x32_10(counter = {i >> 2, s, t, 0}, key = {key0, key1}).
// A launch that draws from the state advances `step` by one when its last workgroup is done (every workgroup reads
// `step` before it reports in `arrivals`, so all of a launch's workgroups see the same value).
#pragma once
#include <cstdint>

namespace niti {

enum : uint32_t { kRngStreamDropout = 1u, kRngStreamLoss = 2u };

__host__ __device__ inline void philox_round(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
  const unsigned long long p0 = 0xD2511F53ULL * c[0];
  const unsigned long long p1 = 0xCD9E8D57ULL * c[2];
  const uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c[1] ^ k0;
  const uint32_t n1 = static_cast<uint32_t>(p1);
  const uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c[3] ^ k1;
  const uint32_t n3 = static_cast<uint32_t>(p0);
  c[0] = n0;
  c[1] = n1;
  c[2] = n2;
  c[3] = n3;
}

__host__ __device__ inline void philox4x32_10(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    philox_round(c, k0, k1);
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

struct RngDraw {
  uint32_t k0, k1, step;
};

__device__ inline RngDraw rng_read(const uint32_t* state) {
  return RngDraw{state[0], state[1], __hip_atomic_load(state + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)};
}

// the four words with indices 4 q .. 4 q + 3 of a stream
__device__ inline void rng_words4(const RngDraw& d, uint32_t stream, uint32_t q, uint32_t (&out)[4]) {
  out[0] = q;
  out[1] = stream;
  out[2] = d.step;
  out[3] = 0u;
  philox4x32_10(out, d.k0, d.k1);
}

__device__ inline uint32_t rng_word(const RngDraw& d, uint32_t stream, uint32_t i) {
  uint32_t w[4];
  rng_words4(d, stream, i >> 2, w);
  return w[i & 3u];
}

// Called by one lane of every workgroup of a launch once the workgroup no longer needs the state (rng_read has
// happened): the last one to arrive starts the next step.
__device__ inline void rng_arrive(uint32_t* state, uint32_t workgroups, const RngDraw& d) {
  const uint32_t seen = __hip_atomic_fetch_add(state + 3, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (seen + 1u == workgroups) {
    __hip_atomic_store(state + 3, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(state + 2, d.step + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace niti
