// Tile bodies of the miniWeather workload: a 2-D stratified-flow solver (finite-volume fluxes with
// fourth-order interface values and hyperviscosity, three-stage Runge-Kutta, x and z sweeps) that
// the reference ships as its non-DNN preemptible workload (src/workloads/miniweather.tr.cu).
// Every kernel of a semi-discrete step is a list of 256-element tiles handed out by the same
// dispatcher as the DNN operators; the in-place state update of the last Runge-Kutta stage is not
// idempotent, which is exactly what "every tile exactly once" has to survive.
//
// Arithmetic follows the reference: fp32 state, x flux formed in fp64 (miniweather.tr.cu:337-348),
// z flux in fp32 (:447-466).  Contraction into fused multiply-adds is switched off in these
// bodies so that results do not depend on how the compiler pairs the operations.
//
// Element ids map to cells as in the reference (:322-324, :382-385, :430-432, :486-489, :511-513,
// :531-533); one lane owns one id, a wavefront reads and writes 256 contiguous bytes per access.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/gpreempt_hip.h"
#include "tile_loop.hpp"

namespace gp {

constexpr int MW_TILE = 256;
constexpr int MW_HS = 2, MW_VARS = 4, MW_DENS = 0, MW_UMOM = 1, MW_WMOM = 2, MW_RHOT = 3;
constexpr float MW_GRAV = 9.8f, MW_C0 = 27.5629410929725921310572974482f, MW_GAMMA = 1.40027894002789400278940027894f;
constexpr float MW_HV_BETA = 0.05f;

__host__ __device__ inline long mw_ids(int kernel, int nx, int nz) {
    switch (kernel) {
        case GP_MW_HALO_X: return (long)nz * MW_VARS;
        case GP_MW_FLUX_X: return (long)nz * (nx + 1);
        case GP_MW_UPDATE_X: return (long)nz * nx * MW_VARS;
        case GP_MW_HALO_Z: return (long)(nx + 2 * MW_HS) * MW_VARS;
        case GP_MW_FLUX_Z: return (long)nx * (nz + 1);
        case GP_MW_UPDATE_Z: return (long)nx * nz * MW_VARS;
    }
    return 0;
}

struct MwView {
    int nx, nz;
    __device__ __forceinline__ long st(int ll, int k, int i) const { return ((long)ll * (nz + 2 * MW_HS) + k) * (nx + 2 * MW_HS) + i; }
    __device__ __forceinline__ long fx(int ll, int k, int i) const { return ((long)ll * (nz + 1) + k) * (nx + 1) + i; }
};

// fourth-order interface value and (scaled) third difference from four cell averages
__device__ __forceinline__ void mw_reconstruct(const float (&s)[4], float hv_coef, float &val, float &d3) {
#pragma clang fp contract(off)
    val = (-s[0] + 7 * (s[1] + s[2]) - s[3]) / 12;
    d3 = (-s[0] + 3 * (s[1] - s[2]) + s[3]) * hv_coef;
}

template <int KIND>
__device__ __forceinline__ void mw_tile(const gp_miniweather_params &p, TileIdx t) {
#pragma clang fp contract(off)
    const MwView v{p.nx, p.nz};
    const int nx = p.nx, nz = p.nz;
    const long id = (long)t.x * MW_TILE + threadIdx.x;
    // hydrostatic background, one buffer: cell density, cell density*theta (nz+4 each), interface
    // density, density*theta, pressure (nz+1 each), four boundary density ratios
    const float *hy_dens_cell = p.hydro, *hy_dens_theta_cell = hy_dens_cell + nz + 2 * MW_HS;
    const float *hy_dens_int = hy_dens_theta_cell + nz + 2 * MW_HS, *hy_dens_theta_int = hy_dens_int + nz + 1;
    const float *hy_pressure_int = hy_dens_theta_int + nz + 1, *hy_cell_const = hy_pressure_int + nz + 1;

    if constexpr (KIND == GP_MW_HALO_X) {  // periodic in x
        const int ll = (int)(id / nz), k = (int)(id % nz);
        if (ll < MW_VARS) {
            float *row = p.state + v.st(ll, k + MW_HS, 0);
            const float a = row[nx + MW_HS - 2], b = row[nx + MW_HS - 1], c = row[MW_HS], d = row[MW_HS + 1];
            row[0] = a; row[1] = b; row[nx + MW_HS] = c; row[nx + MW_HS + 1] = d;
        }
    } else if constexpr (KIND == GP_MW_HALO_Z) {  // solid walls: no flow through, momentum scaled by the density ratio
        const int i = (int)(id % (nx + 2 * MW_HS)), ll = (int)(id / (nx + 2 * MW_HS));
        if (ll < MW_VARS) {
            float *s = p.state;
            if (ll == MW_WMOM) {
                s[v.st(ll, 0, i)] = 0.f; s[v.st(ll, 1, i)] = 0.f;
                s[v.st(ll, nz + MW_HS, i)] = 0.f; s[v.st(ll, nz + MW_HS + 1, i)] = 0.f;
            } else {
                const float lo = s[v.st(ll, MW_HS, i)], hi = s[v.st(ll, nz + MW_HS - 1, i)];
                const bool um = ll == MW_UMOM;
                s[v.st(ll, 0, i)] = um ? lo * hy_cell_const[0] : lo;
                s[v.st(ll, 1, i)] = um ? lo * hy_cell_const[1] : lo;
                s[v.st(ll, nz + MW_HS, i)] = um ? hi * hy_cell_const[2] : hi;
                s[v.st(ll, nz + MW_HS + 1, i)] = um ? hi * hy_cell_const[3] : hi;
            }
        }
    } else if constexpr (KIND == GP_MW_FLUX_X) {
        const int k = (int)(id / (nx + 1)), i = (int)(id % (nx + 1));
        if (k < nz) {
            const float hv_coef = -MW_HV_BETA * p.dx / (16 * p.dt);
            float vals[MW_VARS], d3[MW_VARS];
#pragma unroll
            for (int ll = 0; ll < MW_VARS; ++ll) {
                const float *c = p.state + v.st(ll, k + MW_HS, i);
                const float s[4] = {c[0], c[1], c[2], c[3]};
                mw_reconstruct(s, hv_coef, vals[ll], d3[ll]);
            }
            const double r = vals[MW_DENS] + hy_dens_cell[k + MW_HS];
            const double u = vals[MW_UMOM] / r;
            const double w = vals[MW_WMOM] / r;
            const double th = (vals[MW_RHOT] + hy_dens_theta_cell[k + MW_HS]) / r;
            const double pr = MW_C0 * pow(r * th, (double)MW_GAMMA);
            p.flux[v.fx(MW_DENS, k, i)] = (float)(r * u - d3[MW_DENS]);
            p.flux[v.fx(MW_UMOM, k, i)] = (float)(r * u * u + pr - d3[MW_UMOM]);
            p.flux[v.fx(MW_WMOM, k, i)] = (float)(r * u * w - d3[MW_WMOM]);
            p.flux[v.fx(MW_RHOT, k, i)] = (float)(r * u * th - d3[MW_RHOT]);
        }
    } else if constexpr (KIND == GP_MW_FLUX_Z) {
        const int i = (int)(id % nx), k = (int)(id / nx);
        if (k < nz + 1) {
            const float hv_coef = -MW_HV_BETA * p.dz / (16 * p.dt);
            float vals[MW_VARS], d3[MW_VARS];
#pragma unroll
            for (int ll = 0; ll < MW_VARS; ++ll) {
                const float *c = p.state + v.st(ll, k, i + MW_HS);
                const long row = nx + 2 * MW_HS;
                const float s[4] = {c[0], c[row], c[2 * row], c[3 * row]};
                mw_reconstruct(s, hv_coef, vals[ll], d3[ll]);
            }
            const float r = vals[MW_DENS] + hy_dens_int[k];
            const float u = vals[MW_UMOM] / r;
            float w = vals[MW_WMOM] / r;
            const float th = (vals[MW_RHOT] + hy_dens_theta_int[k]) / r;
            const float pr = MW_C0 * powf(r * th, MW_GAMMA) - hy_pressure_int[k];
            if (k == 0 || k == nz) {  // no flow through the bottom and top faces, exact mass conservation
                w = 0.f;
                d3[MW_DENS] = 0.f;
            }
            p.flux[v.fx(MW_DENS, k, i)] = r * w - d3[MW_DENS];
            p.flux[v.fx(MW_UMOM, k, i)] = r * w * u - d3[MW_UMOM];
            p.flux[v.fx(MW_WMOM, k, i)] = r * w * w + pr - d3[MW_WMOM];
            p.flux[v.fx(MW_RHOT, k, i)] = r * w * th - d3[MW_RHOT];
        }
    } else if constexpr (KIND == GP_MW_UPDATE_X) {
        const int k = (int)((id / nx) % nz), i = (int)(id % nx), ll = (int)(id / nx / nz);
        if (ll < MW_VARS) {
            const float tend = -(p.flux[v.fx(ll, k, i + 1)] - p.flux[v.fx(ll, k, i)]) / p.dx;
            const long c = v.st(ll, k + MW_HS, i + MW_HS);
            p.state_out[c] = p.state_init[c] + p.dt * tend;
        }
    } else {  // GP_MW_UPDATE_Z
        const int i = (int)(id % nx), k = (int)((id / nx) % nz), ll = (int)(id / nx / nz);
        if (ll < MW_VARS) {
            float tend = -(p.flux[v.fx(ll, k + 1, i)] - p.flux[v.fx(ll, k, i)]) / p.dz;
            if (ll == MW_WMOM) {
                // Gravity acts on the density of the forcing state.  When the forcing state is also
                // the output (second Runge-Kutta stage) other lanes overwrite that density in this
                // very kernel; in element order the density ids come first, so the value defined
                // for this read is the UPDATED one, which is recomputed here from operands the
                // kernel never writes instead of being read while it changes.
                const long cd = v.st(MW_DENS, k + MW_HS, i + MW_HS);
                float dens;
                if (p.state == p.state_out) {
                    const float td = -(p.flux[v.fx(MW_DENS, k + 1, i)] - p.flux[v.fx(MW_DENS, k, i)]) / p.dz;
                    dens = p.state_init[cd] + p.dt * td;
                } else {
                    dens = p.state[cd];
                }
                tend = tend - dens * MW_GRAV;
            }
            const long c = v.st(ll, k + MW_HS, i + MW_HS);
            p.state_out[c] = p.state_init[c] + p.dt * tend;
        }
    }
}

template <int KIND>
__global__ __launch_bounds__(MW_TILE) void miniweather_kernel(gp_miniweather_params p, BlpArgs blp) {
    tile_loop(blp, [&](TileIdx t) { mw_tile<KIND>(p, t); });
}

}  // namespace gp
