// Philox4x32-10 counter-based generator (Salmon, Moraes, Dror, Shaw, SC'11) and
// the addressing scheme of the Graph Tsetlin Machine's random decisions.
//
// Every random decision is a pure function of (seed, purpose, clause,
// class/word, training step): the result does not depend on which thread or
// launch shape evaluates it.  The reference instead keeps one cuRAND XORWOW
// state per physical thread (kernels.py:199,228,329,369,643).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define GTM_HD __host__ __device__ __forceinline__
#else
#define GTM_HD static inline
#endif

enum : uint32_t {
    GTM_TAG_PREPARE = 1,         // initial clause weights
    GTM_TAG_CLAUSE_NODE = 2,     // which true node a clause learns from
    GTM_TAG_CLAUSE_UPDATES = 3,  // feedback gates
    GTM_TAG_FEEDBACK = 4,        // Type I feedback bits
};

struct philox_out {
    uint32_t v[4];
};

GTM_HD uint32_t gtm_mulhi32(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __umulhi(a, b);
#else
    return (uint32_t)(((uint64_t)a * (uint64_t)b) >> 32);
#endif
}

GTM_HD philox_out philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
    const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
    const uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        uint32_t hi0 = gtm_mulhi32(M0, c0), lo0 = M0 * c0;
        uint32_t hi1 = gtm_mulhi32(M1, c2), lo1 = M1 * c2;
        uint32_t n0 = hi1 ^ c1 ^ k0;
        uint32_t n2 = hi0 ^ c3 ^ k1;
        c0 = n0;
        c1 = lo1;
        c2 = n2;
        c3 = lo0;
        k0 += W0;
        k1 += W1;
    }
    philox_out out;
    out.v[0] = c0;
    out.v[1] = c1;
    out.v[2] = c2;
    out.v[3] = c3;
    return out;
}

// 32 Bernoulli bits for automaton word `word` of `clause`: bit b is set when
// the b-th 16-bit slice of four Philox blocks is below threshold16
// (threshold16 = min(65536, floor(65536 / s)), so s = 1 gives all ones).
// Stands for the 32 `curand_uniform <= 1/s` draws of kernels.py:113-118,157-162.
GTM_HD uint32_t gtm_feedback_bits(uint32_t k0, uint32_t k1, uint32_t clause, uint32_t word, uint32_t step,
                                  uint32_t bank, uint32_t class_id, uint32_t threshold16) {
    if (threshold16 >= 65536u) return 0xFFFFFFFFu;  // s <= 1: every 16-bit value is below the threshold
    const uint32_t c3 = GTM_TAG_FEEDBACK | (bank << 8) | (class_id << 16);
    uint32_t bits = 0;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        philox_out r = philox4x32_10(clause, word * 4u + j, step, c3, k0, k1);
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            uint32_t lo = r.v[i] & 0xFFFFu, hi = r.v[i] >> 16;
            bits |= (uint32_t)(lo < threshold16) << (j * 8u + i * 2u);
            bits |= (uint32_t)(hi < threshold16) << (j * 8u + i * 2u + 1u);
        }
    }
    return bits;
}
