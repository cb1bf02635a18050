// miniWeather workload: host-side set-up and diagnostics.
//
// Counterpart of the reference's include/workloads/scicomput.h:12-31 (namespaces SciComputeRaw /
// SciComputeBlp: sci_init, reductions, perform_timestep, finalize).  Here the time step is not a
// free function with global state: foo::Model holds the simulation ("miniweather" workload: the
// 36 kernels of one perform_timestep as its kernel list, src/workloads/miniweather.tr.cu:184-206),
// so Executor::execute / BLPExecutor::resume drive it like any DNN and `start_from` is simply the
// stop index.  What remains on the host is below.
#pragma once
#include <cstddef>
#include <vector>

namespace SciCompute {

enum DataSpec { Collision = 1, Thermal = 2, GravityWaves = 3, DensityCurrent = 5, Injection = 6 };

struct Grid {
    int nx, nz;
    float dx, dz, dt;  // dt = min(dx, dz) / 450 * 1.5 (miniweather.tr.cu:584)
};
Grid make_grid(int nx, int nz);

inline size_t state_elems(const Grid &g) { return (size_t)4 * (g.nz + 4) * (g.nx + 4); }
inline size_t flux_elems(const Grid &g) { return (size_t)4 * (g.nz + 1) * (g.nx + 1); }
// cell density, cell density*theta (nz+4 each), interface density, density*theta, pressure (nz+1
// each), four boundary density ratios
inline size_t hydro_elems(const Grid &g) { return (size_t)2 * (g.nz + 4) + 3 * (g.nz + 1) + 4; }

// sci_init (miniweather.tr.cu:555-686): cell averages of the initial perturbation by 3x3
// Gauss-Legendre quadrature and the hydrostatic background columns.
void initial_state(const Grid &g, int data_spec, std::vector<float> &state, std::vector<float> &hydro);

// reductions (miniweather.tr.cu:906-932): domain mass and total energy, accumulated in fp64.
void reductions(const Grid &g, const float *state, const float *hydro, double &mass, double &te);

}  // namespace SciCompute
