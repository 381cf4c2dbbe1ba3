/*
 * comprex_oracle.c -- CPU restatement of ComprEx's compression hot path.
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path, never the product.
 * See comprex_oracle.h for the reference lines each function follows and for
 * how each is pinned.
 *
 * Build: gcc -O3 -DNDEBUG -ffp-contract=off -fPIC -shared (the reference's
 * Release mode, CMakeLists.txt:33; contraction off so that every fp add is the
 * single IEEE add the reference performs).
 */
#include "comprex_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

int cxo_calc_subsamples(float topK, int default_subsamples, float subsample_factor) {
    /* threshold.hxx:183-185.  `cond ? float : int` has type float, so the int
     * operand is rounded to fp32 before the final conversion. */
    float req = subsample_factor / topK;
    float chosen = (req > (float)default_subsamples) ? req : (float)default_subsamples;
    if (!(chosen < 2147483648.0f) || !(chosen > -2147483904.0f)) return -1; /* UB in reference */
    return (int)chosen;
}

int cxo_topk_pos(size_t m, float topK) {
    float prod = (float)m * topK;
    float c = ceilf(prod);
    float r = c - 1.0f;
    return (int)r;
}

int cxo_strided_pos(int i, int n, int subsamples) {
    float stepsize = (float)n / (float)subsamples;
    float x = (float)i * stepsize;
    return (int)x;
}

int cxo_sample_count(int n, int subsamples) {
    return (n < subsamples) ? n : subsamples;
}

#define T float
#define SFX f32
#define ABSV(x) fabsf(x)
#include "comprex_oracle_impl.inc"
#undef T
#undef SFX
#undef ABSV

#define T double
#define SFX f64
#define ABSV(x) fabs(x)
#include "comprex_oracle_impl.inc"
#undef T
#undef SFX
#undef ABSV

#define T int
#define SFX i32
#define ABSV(x) abs(x)
#include "comprex_oracle_impl.inc"
#undef T
#undef SFX
#undef ABSV
