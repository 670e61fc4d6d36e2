/* TEST INFRASTRUCTURE (oracle) -- not part of the product path.
 *
 * Plain C restatement of one timestep of the diffusion/advection stencil program
 * (the module reactant.jl_amd/programs.py:stencil writes, i.e. the slice/compare/select/pad
 * chain Reactant traces from range getindex / ifelse / setindex!: reference src/Indexing.jl:350-445,
 * 552-626, src/Ops.jl:739-792,1865-1930).  Every operation is done in the module's order in
 * double precision and the file is compiled with -ffp-contract=off, so the result has the same
 * bits as the numpy interpreter (tests/test_oracle_golden.py checks that) and as the GPU kernels.
 * Used as the CPU baseline of bench.py on all host cores (OpenMP).
 *
 * Arrays are dense row-major [nz+2H][ny+2H][nx+2H] (Julia dims reversed); the interior is
 * re-embedded in zero halos (`pad`) or written over the previous field (`dus`). */
#include <stddef.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int rx_oracle_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void rx_oracle_stencil_step(const double* c, const double* u, const double* v, const double* w, double* out,
                            int nz, int ny, int nx, int H, double dt, double rdx, double kdx2, int dus) {
  const ptrdiff_t Y = ny + 2 * H, X = nx + 2 * H, Z = nz + 2 * H;
  const ptrdiff_t sy = X, sz = Y * X;
#pragma omp parallel for schedule(static)
  for (ptrdiff_t z = 0; z < Z; ++z) {
    for (ptrdiff_t y = 0; y < Y; ++y) {
      const ptrdiff_t row = z * sz + y * sy;
      const int inside_zy = z >= H && z < H + nz && y >= H && y < H + ny;
      if (!inside_zy) {
        for (ptrdiff_t x = 0; x < X; ++x) out[row + x] = dus ? c[row + x] : 0.0;
        continue;
      }
      for (ptrdiff_t x = 0; x < H; ++x) out[row + x] = dus ? c[row + x] : 0.0;
      for (ptrdiff_t x = H + nx; x < X; ++x) out[row + x] = dus ? c[row + x] : 0.0;
      const double* restrict cr = c + row;
      const double* restrict ur = u + row;
      const double* restrict vr = v + row;
      const double* restrict wr = w + row;
      double* restrict orow = out + row;
      for (ptrdiff_t x = H; x < H + nx; ++x) {
        const double ci = cr[x];
        const double cxm = cr[x - 1], cxp = cr[x + 1], cym = cr[x - sy], cyp = cr[x + sy], czm = cr[x - sz], czp = cr[x + sz];
        double s = cxm + cxp;
        s = s + cym;
        s = s + cyp;
        s = s + czm;
        s = s + czp;
        const double lap = (s - 6.0 * ci) * kdx2;
        const double ax = (ur[x] > 0.0 ? ur[x] * (ci - cxm) : ur[x] * (cxp - ci)) * rdx;
        const double ay = (vr[x] > 0.0 ? vr[x] * (ci - cym) : vr[x] * (cyp - ci)) * rdx;
        const double az = (wr[x] > 0.0 ? wr[x] * (ci - czm) : wr[x] * (czp - ci)) * rdx;
        const double adv = (ax + ay) + az;
        orow[x] = ci + dt * (lap - adv);
      }
    }
  }
}
