/*
 * CPU oracle for the torkit3d point-cloud ops: fp32 and fp64 instantiations of
 * tk3d_oracle_impl.inc.
 *
 * TEST INFRASTRUCTURE ONLY. It exists to check the HIP library and to give the
 * benchmark a CPU figure; the shipped library never links or loads it.
 *
 * Build: see Makefile (gcc -O3 -ffp-contract=off -mfma -fopenmp). Contraction is
 * switched off so that the only fused multiply-adds are the ones written out.
 *
 * How each function is pinned (none is "parity unpinned"):
 *   chamfer fwd   brute force in numpy/torch, identical-cloud and lattice closed
 *                 forms, tie rule on lattice inputs, the known-answer pair in
 *                 tests/ops/test_chamfer_distance.py:42-43 of the reference
 *   chamfer bwd   torch autograd through the brute-force minimum
 *   knn           torch.cdist/topk as sorted (distance, index) pairs, k=1 against
 *                 the chamfer argmin, k=N2 a permutation, slot order against a
 *                 pure-Python MinK on small cases
 *   ball query    numpy nonzero(d2 < r2)[:k] + pad-with-first, r=10 closed form,
 *                 zero-hit rows
 *   fps           numpy running-minimum/argmax recurrence, K=N permutation,
 *                 1-D lattice closed form, a pure-Python thread/tree simulation
 *                 on tie-heavy inputs
 *   group / interpolate   torch.gather, index_add_, autograd
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define REAL float
#define SFX(x) x##_f32
#define FMA fmaf
#include "tk3d_oracle_impl.inc"
#undef REAL
#undef SFX
#undef FMA

#define REAL double
#define SFX(x) x##_f64
#define FMA fma
#include "tk3d_oracle_impl.inc"
#undef REAL
#undef SFX
#undef FMA

#ifdef _OPENMP
#include <omp.h>
#endif

/* Threads the parallel loops will use (1 when built without OpenMP). */
int tk3d_oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void tk3d_oracle_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0)
        omp_set_num_threads(n);
#else
    (void)n;
#endif
}
