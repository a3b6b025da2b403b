/* Native host-side encoder of node properties into the literal words of X.
 *
 * The reference encodes one property per Python call, through a numba loop
 * (GraphTsetlinMachine/graphs.py:148-162): for every hypervector index k of the
 * symbol, set literal k and clear its negation k + hypervector_size in the
 * node's row.  Data sets with 10^9 property insertions cannot be built that
 * way; these two entry points are the same loop over whole arrays, spread over
 * OpenMP threads.  Plain C (gcc), loaded by graphs.py through ctypes; results
 * are bit-identical to repeated single calls.
 *
 * X is uint32 [rows][chunks]; hypervectors uint32 [symbols][bits].
 */
#include <stdint.h>

static inline void add_symbol(uint32_t *row, const uint32_t *indices, int bits, int hv_size) {
    for (int j = 0; j < bits; ++j) {
        const uint32_t k = indices[j], n = k + (uint32_t)hv_size;
        row[k >> 5] |= 1u << (k & 31);
        row[n >> 5] &= ~(1u << (n & 31));
    }
}

/* membership[r][s] != 0 adds symbol s to row r of X (X points at the first of the n_rows rows).
 * Rows are independent: one thread per run of rows. */
void gtm_encode_membership(const uint8_t *membership, int64_t n_rows, int32_t n_symbols, const uint32_t *hypervectors,
                           int32_t bits, int32_t hv_size, int32_t chunks, uint32_t *X) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n_rows; ++r) {
        const uint8_t *m = membership + r * n_symbols;
        uint32_t *row = X + r * chunks;
        for (int32_t s = 0; s < n_symbols; ++s)
            if (m[s]) add_symbol(row, hypervectors + (int64_t)s * bits, bits, hv_size);
    }
}

/* Pair i adds symbol symbols[i] to row rows[i] (global node rows).  Pairs may repeat and come in
 * any order; threads may meet on a row, so the word updates are atomic (setting and clearing bits
 * commute, and no pair sets what another clears: a literal is set, its negation cleared). */
void gtm_encode_pairs(const int64_t *rows, const int64_t *symbols, int64_t n_pairs, const uint32_t *hypervectors,
                      int32_t bits, int32_t hv_size, int32_t chunks, uint32_t *X) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n_pairs; ++i) {
        uint32_t *row = X + rows[i] * chunks;
        const uint32_t *indices = hypervectors + symbols[i] * bits;
        for (int j = 0; j < bits; ++j) {
            const uint32_t k = indices[j], n = k + (uint32_t)hv_size;
            __atomic_fetch_or(&row[k >> 5], 1u << (k & 31), __ATOMIC_RELAXED);
            __atomic_fetch_and(&row[n >> 5], ~(1u << (n & 31)), __ATOMIC_RELAXED);
        }
    }
}
