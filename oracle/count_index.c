/*
 * CPU oracle, integer part, in plain C: TEST INFRASTRUCTURE, not product code (only tests/, the smoke check and the
 * cpu_baseline leg of bench.py load it). It restates, one element at a time, what the reference computes:
 *
 *  oracle_continuous_count_*: the histogram of fma/ops/continuous_count/__init__.py:29-36
 *      (`x.bincount(minlength=size).to(uint32)`); its CUDA kernel does the same with one shared-memory atomicAdd per
 *      element (cuda_implementation/forward.cu:50-70). Values outside [0, size) are skipped (docstring :15-17).
 *  oracle_routing_index: `selected_experts.flatten().sort()` + counts + `cumsum(-1)`
 *      (fma/modules/moe/__init__.py:214-217,249) as a counting sort; slots of one expert stay in ascending order
 *      (the order of torch.sort(stable=True)).
 *
 * Pinned in tests/test_oracle.py against numpy.bincount, torch.sort(stable=True) and the numpy restatement.
 * Build: gcc -O2 -shared -fPIC oracle/count_index.c -o oracle/_build/liboracle.so  (see oracle/build.py)
 */
#include <stdint.h>
#include <string.h>

void oracle_continuous_count_i32(const int32_t* x, uint64_t n, uint32_t size, uint32_t* out) {
    memset(out, 0, (size_t)size * sizeof(uint32_t));
    for (uint64_t i = 0; i < n; ++i) {
        const int32_t v = x[i];
        if (v >= 0 && (uint32_t)v < size) out[v] += 1;
    }
}

void oracle_continuous_count_i64(const int64_t* x, uint64_t n, uint32_t size, uint32_t* out) {
    memset(out, 0, (size_t)size * sizeof(uint32_t));
    for (uint64_t i = 0; i < n; ++i) {
        const int64_t v = x[i];
        if (v >= 0 && v < (int64_t)size) out[v] += 1;
    }
}

/* ids: R expert ids in [0, E). counts/offsets: E entries; perm/eid/inv: R entries; cursor: scratch of E entries. */
void oracle_routing_index(const int64_t* ids, int64_t R, uint32_t E, uint32_t* counts, uint32_t* offsets,
                          int32_t* perm, int32_t* eid, int32_t* inv, uint32_t* cursor) {
    oracle_continuous_count_i64(ids, (uint64_t)R, E, counts);
    uint32_t running = 0;
    for (uint32_t e = 0; e < E; ++e) {
        cursor[e] = running; /* first output row of expert e */
        running += counts[e];
        offsets[e] = running; /* inclusive prefix */
    }
    for (int64_t s = 0; s < R; ++s) {
        const int64_t e = ids[s];
        const uint32_t pos = cursor[e]++;
        perm[pos] = (int32_t)s;
        eid[pos] = (int32_t)e;
        inv[s] = (int32_t)pos;
    }
}
