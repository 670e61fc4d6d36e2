/* TEST INFRASTRUCTURE (oracle) -- not part of the product path.
 *
 * Plain C restatement of the sinsum_add program, sum(sin.(x) .+ y) over Float32 vectors (the module
 * reactant.jl_amd/programs.py:sinsum_add writes: stablehlo.sine, add, reduce; reference src/Ops.jl:739-792
 * for the elementwise ops and src/TracedRArray.jl mapreduce for the reduction).  Each term is formed in single
 * precision as the module does; the terms are summed in double precision (the order of a parallel sum is not
 * part of the program's meaning, and the double sum is within 1e-12 of exact for 2^26 terms).
 * Used as the CPU baseline of bench.py on all host cores (OpenMP) and pinned against numpy in
 * tests/test_oracle_golden.py. */
#include <math.h>
#include <stddef.h>

double rx_oracle_sinsum_add(const float* x, const float* y, long long n) {
  double s = 0.0;
#pragma omp parallel for schedule(static) reduction(+ : s)
  for (long long i = 0; i < n; ++i) {
    const float t = sinf(x[i]) + y[i];
    s += (double)t;
  }
  return s;
}
