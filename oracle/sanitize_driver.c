/* Test infrastructure: drives the C restatement of the integer pipeline (routing_oracle.c) under the host
 * AddressSanitizer / UndefinedBehaviorSanitizer build (`make -C oracle asan`).  Exact-size heap buffers, so that any
 * access past an end is reported; results are also checked against definitions (stable order, histogram, running
 * sums, block table) so the run fails on a wrong answer as well as on a sanitizer report.  Exit code 0 = clean. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

int oracle_topk_renorm(const float* scores, int64_t T, int E, int k, int renorm, int32_t* idx, float* w);
int oracle_sort_by_expert(const int32_t* expert_idx, int64_t R, int E, int32_t* sorted_expert, int32_t* sorted_pos,
                          int32_t* counts, int32_t* offsets, int32_t* inv);
int64_t oracle_padded_block_indices(const int32_t* sorted_expert, int64_t R, int E, int block_m, int32_t* blocks,
                                    int64_t cap, int32_t* offsets);

static uint32_t rng_state = 12345u;
static uint32_t rnd(void) { rng_state = rng_state * 1664525u + 1013904223u; return rng_state >> 8; }

#define CHECK(c) do { if (!(c)) { fprintf(stderr, "check failed: %s (line %d, R=%lld E=%d)\n", #c, __LINE__, (long long)R, E); return 1; } } while (0)

static int sort_case(int64_t R, int E, int block_m, int skew)
{
    int32_t* in = malloc((size_t)(R ? R : 1) * 4), *se = malloc((size_t)(R ? R : 1) * 4), *sp = malloc((size_t)(R ? R : 1) * 4);
    int32_t* inv = malloc((size_t)(R ? R : 1) * 4), *counts = malloc((size_t)E * 4), *offs = malloc((size_t)E * 4), *offs2 = malloc((size_t)E * 4);
    const int64_t cap = R / block_m + E;
    int32_t* blocks = malloc((size_t)(cap ? cap : 1) * 4);
    for (int64_t i = 0; i < R; ++i) in[i] = skew ? (int32_t)((rnd() % 7) ? 0 : rnd() % (uint32_t)E) : (int32_t)(rnd() % (uint32_t)E);
    CHECK(oracle_sort_by_expert(in, R, E, se, sp, counts, offs, inv) == 0);
    int64_t run = 0;
    for (int e = 0; e < E; ++e) { run += counts[e]; CHECK(offs[e] == run); }
    CHECK(run == R);
    for (int64_t i = 0; i < R; ++i) {
        CHECK(sp[i] >= 0 && sp[i] < R && in[sp[i]] == se[i] && inv[sp[i]] == i);
        if (i) CHECK(se[i - 1] < se[i] || (se[i - 1] == se[i] && sp[i - 1] < sp[i]));   /* stable ascending */
    }
    const int64_t nb = oracle_padded_block_indices(se, R, E, block_m, blocks, cap, offs2);
    CHECK(nb >= 0 && nb <= cap);
    int64_t want = 0, b = 0, start = 0;
    for (int e = 0; e < E; ++e) {
        CHECK(offs2[e] == offs[e]);
        for (int64_t s = start; s < offs[e]; s += block_m, ++b) CHECK(blocks[b] == s);
        want += (offs[e] - start + block_m - 1) / block_m;
        start = offs[e];
    }
    CHECK(nb == want && b == nb);
    free(in); free(se); free(sp); free(inv); free(counts); free(offs); free(offs2); free(blocks);
    return 0;
}

static int topk_case(int64_t R /* tokens */, int E, int k, int renorm)
{
    float* sc = malloc((size_t)(R ? R : 1) * (size_t)E * 4), *w = malloc((size_t)(R ? R : 1) * (size_t)k * 4);
    int32_t* idx = malloc((size_t)(R ? R : 1) * (size_t)k * 4);
    for (int64_t i = 0; i < R * E; ++i) sc[i] = (float)(rnd() % 16) / 16.0f + 1e-3f;   /* coarse values: plenty of ties */
    CHECK(oracle_topk_renorm(sc, R, E, k, renorm, idx, w) == 0);
    for (int64_t t = 0; t < R; ++t) {
        float sum = 0.f;
        for (int j = 0; j < k; ++j) {
            const int32_t e = idx[t * k + j];
            CHECK(e >= 0 && e < E);
            for (int j2 = 0; j2 < j; ++j2) CHECK(idx[t * k + j2] != e);
            if (j) {   /* descending score, ties to the lower expert id */
                const float prev = sc[t * E + idx[t * k + j - 1]], cur = sc[t * E + e];
                CHECK(prev > cur || (prev == cur && idx[t * k + j - 1] < e));
            }
            sum += w[t * k + j];
        }
        if (renorm) CHECK(sum > 0.999f && sum < 1.001f);
    }
    free(sc); free(w); free(idx);
    return 0;
}

int main(void)
{
    const int64_t Rs[] = {0, 1, 2, 10, 127, 128, 129, 1000, 8192, 40001};
    const int Es[] = {1, 2, 3, 8, 64, 257};
    for (unsigned a = 0; a < sizeof Rs / sizeof *Rs; ++a)
        for (unsigned b = 0; b < sizeof Es / sizeof *Es; ++b)
            for (int skew = 0; skew < 2; ++skew)
                if (sort_case(Rs[a], Es[b], (a & 1) ? 128 : 7, skew)) return 1;
    const int Ek[][2] = {{1, 1}, {2, 1}, {2, 2}, {8, 2}, {8, 8}, {64, 6}, {1024, 3}};
    for (unsigned a = 0; a < sizeof Ek / sizeof *Ek; ++a)
        for (int renorm = 0; renorm < 2; ++renorm) {
            if (topk_case(0, Ek[a][0], Ek[a][1], renorm)) return 1;
            if (topk_case(301, Ek[a][0], Ek[a][1], renorm)) return 1;
        }
    { int64_t R = 0; int E = 4; int32_t i4[4] = {0}; float f4[4] = {0}; CHECK(oracle_topk_renorm(f4, 1, E, 5, 1, i4, f4) == -1); }   /* k > E is refused */
    printf("routing oracle: sanitizer run clean\n");
    return 0;
}
