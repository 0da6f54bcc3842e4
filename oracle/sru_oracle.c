/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU oracle for the SRU elementwise recurrence (forward scan and analytic
 * backward scan). Nothing shipped links or calls this file: it is built into
 * liboracle.so by the Makefile beside it and loaded only by the tests, by the
 * smoke check and by the CPU-baseline leg of the benchmark.
 *
 * Two instantiations of sru_oracle_impl.h:
 *   *_f32  arithmetic in float, expf/tanhf: what the reference's serial CPU loop
 *          (sru/csrc/sru_cpu_impl.cpp:56-226) computes, plus the backward
 *          equations of sru/csrc/sru_cuda_kernel.cu:447-578,:667-822.
 *   *_f64  the same in double: the checker.
 *
 * What pins it (see tests/test_oracle_*.py): the reference's golden vector
 * test/regression/artifacts/2.3.5.pt, the reference's own CPU routine compiled
 * from its source (oracle/_ref), gradcheck / finite differences for the backward
 * equations, and closed forms (weight_c = 0, saturated gates).
 */
#include <math.h>
#include <stdint.h>

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define REAL float
#define FN(name) CAT(name, _f32)
#define EXP expf
#define TANH tanhf
#include "sru_oracle_impl.h"
#undef REAL
#undef FN
#undef EXP
#undef TANH

#define REAL double
#define FN(name) CAT(name, _f64)
#define EXP exp
#define TANH tanh
#include "sru_oracle_impl.h"
#undef REAL
#undef FN
#undef EXP
#undef TANH
