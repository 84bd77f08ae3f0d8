// The library's random stream: Philox4x32-10, shared by every kernel that draws uniforms.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace dbk_rng {

// Philox4x32-10 counter-based generator (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3").
// One 128-bit counter value yields four 32-bit words; element i uses word i%4 of counter (offset + i/4).
__host__ __device__ inline void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1)
{
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
}

// Uniform in [0,1) with 24 bits, for flat element index i.
__device__ inline float uniform_at(uint64_t seed, uint64_t offset, size_t i)
{
    uint64_t ctr = offset + (uint64_t)(i >> 2);
    uint32_t c[4] = {(uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u};
    philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
    return (float)(c[i & 3] >> 8) * (1.0f / 16777216.0f);
}

// The four uniforms of flat elements 4q .. 4q+3 (one generator call).
__device__ inline void uniform4_at(uint64_t seed, uint64_t offset, size_t q, float u[4])
{
    uint64_t ctr = offset + (uint64_t)q;
    uint32_t c[4] = {(uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u};
    philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
#pragma unroll
    for (int j = 0; j < 4; ++j) u[j] = (float)(c[j] >> 8) * (1.0f / 16777216.0f);
}

}  // namespace dbk_rng
