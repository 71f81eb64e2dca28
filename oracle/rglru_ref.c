/* Plain-C CPU oracle for the Conv1D + RG-LRU hot path, in float and double.
 *
 * TEST INFRASTRUCTURE ONLY (see rglru_ref_impl.h).  Built by `make -C oracle`
 * into oracle/librglru_ref.so and loaded with ctypes by the tests, the smoke
 * check and the benchmark's CPU-baseline leg.
 *
 * Exported symbols: ref_<fn>_f32 and ref_<fn>_f64 for
 *   conv1d_prefill, conv1d_step, block_diag_linear, rglru_scan.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#define REAL float
#define SUFFIX(n) n##_f32
#define R_EXP expf
#define R_LOG1P log1pf
#define R_SQRT sqrtf
#include "rglru_ref_impl.h"
#undef REAL
#undef SUFFIX
#undef R_EXP
#undef R_LOG1P
#undef R_SQRT

#define REAL double
#define SUFFIX(n) n##_f64
#define R_EXP exp
#define R_LOG1P log1p
#define R_SQRT sqrt
#include "rglru_ref_impl.h"
