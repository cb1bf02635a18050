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

// Pointers into the hydrostatic background buffer: cell density, cell density*theta (nz+4 each),
// interface density, density*theta, pressure (nz+1 each), four boundary density ratios.
struct MwHydro {
    const float *dens_cell, *dens_theta_cell, *dens_int, *dens_theta_int, *pressure_int, *cell_const;
    __device__ __forceinline__ MwHydro(const float *h, int nz) {
        dens_cell = h;
        dens_theta_cell = dens_cell + nz + 2 * MW_HS;
        dens_int = dens_theta_cell + nz + 2 * MW_HS;
        dens_theta_int = dens_int + nz + 1;
        pressure_int = dens_theta_int + nz + 1;
        cell_const = pressure_int + nz + 1;
    }
};

// What one element id reads, split from what it computes and writes so that a lane can have the
// loads of several ids in flight before the first result is needed (an id alone keeps 12-72 bytes
// in flight per lane, too few to cover HBM latency at 32 waves per CU).
template <int KIND> struct MwOperands;

template <> struct MwOperands<GP_MW_UPDATE_X> { long c; float f0, f1, init; };
template <> struct MwOperands<GP_MW_UPDATE_Z> { long c; int ll; float f0, f1, init, d0, d1, dinit; };
template <> struct MwOperands<GP_MW_FLUX_X> { int k, i; float s[MW_VARS][4], h0, h1; };
template <> struct MwOperands<GP_MW_FLUX_Z> { int k, i; float s[MW_VARS][4], h0, h1, h2; };

__device__ __forceinline__ bool mw_load(const gp_miniweather_params &p, unsigned id, MwOperands<GP_MW_UPDATE_X> &o) {
    const MwView v{p.nx, p.nz};
    const unsigned nx = p.nx, nz = p.nz;
    const unsigned row = id / nx;  // 32-bit: ids stay below 2^29 (the launcher bounds nx * nz)
    const int i = (int)(id - row * nx), ll = (int)(row / nz), k = (int)(row - (unsigned)ll * nz);
    if (ll >= MW_VARS) return false;
    o.c = v.st(ll, k + MW_HS, i + MW_HS);
    o.f0 = p.flux[v.fx(ll, k, i)];
    o.f1 = p.flux[v.fx(ll, k, i + 1)];
    o.init = p.state_init[o.c];
    return true;
}
__device__ __forceinline__ void mw_finish(const gp_miniweather_params &p, const MwOperands<GP_MW_UPDATE_X> &o) {
#pragma clang fp contract(off)
    const float tend = -(o.f1 - o.f0) / p.dx;
    p.state_out[o.c] = o.init + p.dt * tend;
}

__device__ __forceinline__ bool mw_load(const gp_miniweather_params &p, unsigned id, MwOperands<GP_MW_UPDATE_Z> &o) {
    const MwView v{p.nx, p.nz};
    const unsigned nx = p.nx, nz = p.nz;
    const unsigned row = id / nx;
    const int i = (int)(id - row * nx), ll = (int)(row / nz), k = (int)(row - (unsigned)ll * nz);
    if (ll >= MW_VARS) return false;
    o.ll = ll;
    o.c = v.st(ll, k + MW_HS, i + MW_HS);
    o.f0 = p.flux[v.fx(ll, k, i)];
    o.f1 = p.flux[v.fx(ll, k + 1, i)];
    o.init = p.state_init[o.c];
    o.d0 = o.d1 = o.dinit = 0.f;
    if (ll == MW_WMOM) {
        // Gravity acts on the density of the forcing state.  When the forcing state is also the
        // output (second Runge-Kutta stage) other lanes overwrite that density in this very
        // kernel; in element order the density ids come first, so the value defined for this read
        // is the UPDATED one, which is recomputed from operands the kernel never writes instead
        // of being read while it changes.
        const long cd = v.st(MW_DENS, k + MW_HS, i + MW_HS);
        if (p.state == p.state_out) {
            o.d0 = p.flux[v.fx(MW_DENS, k, i)];
            o.d1 = p.flux[v.fx(MW_DENS, k + 1, i)];
            o.dinit = p.state_init[cd];
        } else {
            o.dinit = p.state[cd];
        }
    }
    return true;
}
__device__ __forceinline__ void mw_finish(const gp_miniweather_params &p, const MwOperands<GP_MW_UPDATE_Z> &o) {
#pragma clang fp contract(off)
    float tend = -(o.f1 - o.f0) / p.dz;
    if (o.ll == MW_WMOM) {
        float dens = o.dinit;
        if (p.state == p.state_out) {
            const float td = -(o.d1 - o.d0) / p.dz;
            dens = o.dinit + p.dt * td;
        }
        tend = tend - dens * MW_GRAV;
    }
    p.state_out[o.c] = o.init + p.dt * tend;
}

__device__ __forceinline__ bool mw_load(const gp_miniweather_params &p, unsigned id, MwOperands<GP_MW_FLUX_X> &o) {
    const MwView v{p.nx, p.nz};
    const MwHydro hy(p.hydro, p.nz);
    const unsigned w = p.nx + 1;
    o.k = (int)(id / w);
    o.i = (int)(id - (unsigned)o.k * w);
    if (o.k >= p.nz) return false;
#pragma unroll
    for (int ll = 0; ll < MW_VARS; ++ll) {
        const float *c = p.state + v.st(ll, o.k + MW_HS, o.i);
#pragma unroll
        for (int s = 0; s < 4; ++s) o.s[ll][s] = c[s];
    }
    o.h0 = hy.dens_cell[o.k + MW_HS];
    o.h1 = hy.dens_theta_cell[o.k + MW_HS];
    return true;
}
__device__ __forceinline__ void mw_finish(const gp_miniweather_params &p, const MwOperands<GP_MW_FLUX_X> &o) {
#pragma clang fp contract(off)
    const MwView v{p.nx, p.nz};
    const float hv_coef = -MW_HV_BETA * p.dx / (16 * p.dt);
    float vals[MW_VARS], d3[MW_VARS];
#pragma unroll
    for (int ll = 0; ll < MW_VARS; ++ll) mw_reconstruct(o.s[ll], hv_coef, vals[ll], d3[ll]);
    const double r = vals[MW_DENS] + o.h0;
    const double u = vals[MW_UMOM] / r;
    const double w = vals[MW_WMOM] / r;
    const double th = (vals[MW_RHOT] + o.h1) / r;
    // (rho theta)^gamma as exp(gamma log(.)): the argument is positive and the result is rounded to
    // fp32 when the flux is stored, 8 decimal digits above what the fp64 exp/log pair loses, and
    // the pair costs a third of a general pow (which made this kernel ALU-bound: 60 us of fp64
    // work against 35 us of memory traffic)
    const double pr = MW_C0 * exp((double)MW_GAMMA * log(r * th));
    p.flux[v.fx(MW_DENS, o.k, o.i)] = (float)(r * u - d3[MW_DENS]);
    p.flux[v.fx(MW_UMOM, o.k, o.i)] = (float)(r * u * u + pr - d3[MW_UMOM]);
    p.flux[v.fx(MW_WMOM, o.k, o.i)] = (float)(r * u * w - d3[MW_WMOM]);
    p.flux[v.fx(MW_RHOT, o.k, o.i)] = (float)(r * u * th - d3[MW_RHOT]);
}

__device__ __forceinline__ bool mw_load(const gp_miniweather_params &p, unsigned id, MwOperands<GP_MW_FLUX_Z> &o) {
    const MwView v{p.nx, p.nz};
    const MwHydro hy(p.hydro, p.nz);
    const int nx = p.nx;
    o.k = (int)(id / (unsigned)nx);
    o.i = (int)(id - (unsigned)o.k * (unsigned)nx);
    if (o.k >= p.nz + 1) return false;
    const long row = nx + 2 * MW_HS;
#pragma unroll
    for (int ll = 0; ll < MW_VARS; ++ll) {
        const float *c = p.state + v.st(ll, o.k, o.i + MW_HS);
#pragma unroll
        for (int s = 0; s < 4; ++s) o.s[ll][s] = c[s * row];
    }
    o.h0 = hy.dens_int[o.k];
    o.h1 = hy.dens_theta_int[o.k];
    o.h2 = hy.pressure_int[o.k];
    return true;
}
__device__ __forceinline__ void mw_finish(const gp_miniweather_params &p, const MwOperands<GP_MW_FLUX_Z> &o) {
#pragma clang fp contract(off)
    const MwView v{p.nx, p.nz};
    const float hv_coef = -MW_HV_BETA * p.dz / (16 * p.dt);
    float vals[MW_VARS], d3[MW_VARS];
#pragma unroll
    for (int ll = 0; ll < MW_VARS; ++ll) mw_reconstruct(o.s[ll], hv_coef, vals[ll], d3[ll]);
    const float r = vals[MW_DENS] + o.h0;
    const float u = vals[MW_UMOM] / r;
    float w = vals[MW_WMOM] / r;
    const float th = (vals[MW_RHOT] + o.h1) / r;
    const float pr = MW_C0 * powf(r * th, MW_GAMMA) - o.h2;
    if (o.k == 0 || o.k == p.nz) {  // no flow through the bottom and top faces, exact mass conservation
        w = 0.f;
        d3[MW_DENS] = 0.f;
    }
    p.flux[v.fx(MW_DENS, o.k, o.i)] = r * w - d3[MW_DENS];
    p.flux[v.fx(MW_UMOM, o.k, o.i)] = r * w * u - d3[MW_UMOM];
    p.flux[v.fx(MW_WMOM, o.k, o.i)] = r * w * w + pr - d3[MW_WMOM];
    p.flux[v.fx(MW_RHOT, o.k, o.i)] = r * w * th - d3[MW_RHOT];
}

// halo kernels: a few thousand ids, nothing to overlap
template <int KIND>
__device__ __forceinline__ void mw_halo(const gp_miniweather_params &p, long id) {
#pragma clang fp contract(off)
    const MwView v{p.nx, p.nz};
    const int nx = p.nx, nz = p.nz;
    if constexpr (KIND == GP_MW_HALO_X) {  // periodic in x
        const int ll = (int)(id / nz), k = (int)(id % nz);
        if (ll < MW_VARS) {
            float *row = p.state + v.st(ll, k + MW_HS, 0);
            const float a = row[nx + MW_HS - 2], b = row[nx + MW_HS - 1], c = row[MW_HS], d = row[MW_HS + 1];
            row[0] = a; row[1] = b; row[nx + MW_HS] = c; row[nx + MW_HS + 1] = d;
        }
    } else {  // solid walls: no flow through, horizontal momentum scaled by the density ratio
        const MwHydro hy(p.hydro, nz);
        const int i = (int)(id % (nx + 2 * MW_HS)), ll = (int)(id / (nx + 2 * MW_HS));
        if (ll < MW_VARS) {
            float *s = p.state;
            if (ll == MW_WMOM) {
                s[v.st(ll, 0, i)] = 0.f; s[v.st(ll, 1, i)] = 0.f;
                s[v.st(ll, nz + MW_HS, i)] = 0.f; s[v.st(ll, nz + MW_HS + 1, i)] = 0.f;
            } else {
                const float lo = s[v.st(ll, MW_HS, i)], hi = s[v.st(ll, nz + MW_HS - 1, i)];
                const bool um = ll == MW_UMOM;
                s[v.st(ll, 0, i)] = um ? lo * hy.cell_const[0] : lo;
                s[v.st(ll, 1, i)] = um ? lo * hy.cell_const[1] : lo;
                s[v.st(ll, nz + MW_HS, i)] = um ? hi * hy.cell_const[2] : hi;
                s[v.st(ll, nz + MW_HS + 1, i)] = um ? hi * hy.cell_const[3] : hi;
            }
        }
    }
}

// Tiles [first, last) of one claim: U tiles at a time, all loads first.  The ids of different
// tiles never touch the same output element, and an update reads the element it writes only
// through its own lane, so issuing the loads of U tiles ahead of their stores changes nothing.
template <int KIND>
__device__ __forceinline__ void mw_span(const gp_miniweather_params &p, int first, int last) {
    if constexpr (KIND == GP_MW_HALO_X || KIND == GP_MW_HALO_Z) {
        for (int t = first; t < last; ++t) mw_halo<KIND>(p, (long)t * MW_TILE + threadIdx.x);
    } else {
        constexpr int U = (KIND == GP_MW_UPDATE_X || KIND == GP_MW_UPDATE_Z) ? 4 : 2;
        for (int t = first; t < last; t += U) {
            MwOperands<KIND> op[U];
            bool ok[U];
#pragma unroll
            for (int j = 0; j < U; ++j) ok[j] = t + j < last && mw_load(p, (unsigned)(t + j) * MW_TILE + threadIdx.x, op[j]);
#pragma unroll
            for (int j = 0; j < U; ++j)
                if (ok[j]) mw_finish(p, op[j]);
        }
    }
}

template <int KIND, int LOOP = LOOP_ANY>
__global__ __launch_bounds__(MW_TILE) void miniweather_kernel(gp_miniweather_params p, BlpArgs blp) {
    spans<LOOP>(blp, [&](int first, int last) { mw_span<KIND>(p, first, last); });
}

}  // namespace gp
