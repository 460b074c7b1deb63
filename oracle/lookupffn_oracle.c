/*
 * TEST INFRASTRUCTURE ONLY.  A plain-C CPU restatement of the reference's
 * LookupFFN hot path (FHT / BH4 projection, code+score, weighted gather-add and
 * its backward, whole layer), used as the checker by the tests, the smoke test
 * and the bench's CPU-baseline leg.  Nothing in the product package may link,
 * load or call it.
 *
 * Every function is instantiated as <name>_f32 (the reference's arithmetic,
 * in the reference's operation order) and <name>_f64 (truth for tolerances).
 * Built with -ffp-contract=off so that the f32 results are plain IEEE
 * mul-then-add, independent of the host's FMA support.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   orc_fht              x @ scipy.linalg.hadamard(D) (the reference's own check,
 *                        fast_hadamard_transform/kernel.py:31-37), exact on integer
 *                        inputs; H.H = D.I; brute force D <= 64
 *   orc_bh4 / projection torch.einsum("bni,noi->bno") + scipy Hadamard composition
 *   orc_code_score       exhaustive 2^8 sign patterns, brute-force bit loop, special
 *                        values (0, -0, NaN), fp64 closed form, and the reference's
 *                        own x86 kernel where oracle/_ref is built
 *   orc_code_score_bwd   torch.autograd of the reference formula (float64)
 *   orc_gather_add       torch.nn.functional.embedding_bag, one-hot/constant-table
 *                        cases, and the reference's x86 kernels where oracle/_ref is built
 *   orc_gather_add_bf16  the f32 routine on the widened table (exact widening)
 *   orc_indexed_inner_product / orc_scatter_add
 *                        torch autograd of embedding_bag and the reference's slow formulas
 *   orc_layernorm        torch.nn.functional.layer_norm
 *   orc_lookup_ffn       composition of the pinned parts in torch
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define REAL float
#define FN(name) CAT(name, _f32)
#define ABS fabsf
#define EXP expf
#define SQRT sqrtf
#include "lookupffn_oracle_impl.h"
#undef REAL
#undef FN
#undef ABS
#undef EXP
#undef SQRT

#define REAL double
#define FN(name) CAT(name, _f64)
#define ABS fabs
#define EXP exp
#define SQRT sqrt
#include "lookupffn_oracle_impl.h"
#undef REAL
#undef FN
#undef ABS
#undef EXP
#undef SQRT

int orc_version(void) { return 1; }

/* Threads the parallel loops above use (for reporting the CPU baseline). */
#ifdef _OPENMP
#include <omp.h>
int orc_num_threads(void) { return omp_get_max_threads(); }
#else
int orc_num_threads(void) { return 1; }
#endif
