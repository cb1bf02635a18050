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

// x / 12 with the bits of the division (checked against it on 1.5 * 10^7 random floats): the product with the rounded
// reciprocal, corrected by the exact remainder.  Three instructions for the eleven of an fp32 division, in kernels
// whose time is the number of vector instructions they issue per cell.
__device__ __forceinline__ float mw_div12(float x) {
    const float c = 1.0f / 12.0f;
    const float q = x * c;
    const float r = __builtin_fmaf(-q, 12.0f, x);
    return __builtin_fmaf(r, c, q);
}

// The (row, column) of a claim's ids in rows of w ids: one division per claim, then additions, instead of a
// division per id (twenty vector instructions).
struct MwCursor {
    unsigned w, i;
    int k;
    __device__ __forceinline__ MwCursor(unsigned id0, unsigned w_) : w(w_) { k = (int)(id0 / w); i = id0 - (unsigned)k * w; }
    __device__ __forceinline__ void next_tile() {
        i += MW_TILE;
        while (i >= w) { i -= w; ++k; }
    }
    __device__ __forceinline__ void lane(int &kl, int &il) const {
        unsigned x = i + threadIdx.x;
        int kk = k;
        while (x >= w) { x -= w; ++kk; }
        kl = kk; il = (int)x;
    }
};

// fourth-order interface value and (scaled) third difference from four cell averages
__device__ __forceinline__ void mw_reconstruct(const float (&s)[4], float hv_coef, float &val, float &d3) {
#pragma clang fp contract(off)
    val = mw_div12(-s[0] + 7 * (s[1] + s[2]) - s[3]);
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

template <> struct MwOperands<GP_MW_UPDATE_X> { unsigned c; float f0, f1, init; };
template <> struct MwOperands<GP_MW_UPDATE_Z> { unsigned c; int ll; float f0, f1, init, d0, d1, dinit; };
template <> struct MwOperands<GP_MW_FLUX_X> { int k, i; float s[MW_VARS][4], h0, h1; };
template <> struct MwOperands<GP_MW_FLUX_Z> { int k, i; float s[MW_VARS][4], h0, h1, h2; };

// a / b from the correctly rounded reciprocal c of b: the product, corrected by its exact remainder, which is the
// rounded quotient itself (Markstein's sequence; three instructions for the eleven of an fp32 division)
__device__ __forceinline__ float mw_div(float a, float b, float c) {
    const float q = a * c;
    const float r = __builtin_fmaf(-q, b, a);
    return __builtin_fmaf(r, c, q);
}
// an update id is (field, level, column): the cursor gives field * nz + level and the column
__device__ __forceinline__ bool mw_update_cell(const gp_miniweather_params &p, const MwCursor &cur, int &ll, int &k, int &i) {
    int row;
    cur.lane(row, i);
    const int nz = p.nz;
    if (row >= MW_VARS * nz) return false;
    ll = (row >= nz) + (row >= 2 * nz) + (row >= 3 * nz);
    k = row - ll * nz;
    return true;
}
__device__ __forceinline__ bool mw_load(const gp_miniweather_params &p, const MwCursor &cur, MwOperands<GP_MW_UPDATE_X> &o) {
    int ll, k, i;
    if (!mw_update_cell(p, cur, ll, k, i)) return false;
    o.c = (unsigned)(ll * (p.nz + 2 * MW_HS) + k + MW_HS) * (unsigned)(p.nx + 2 * MW_HS) + (unsigned)(i + MW_HS);
    const unsigned f = (unsigned)(ll * (p.nz + 1) + k) * (unsigned)(p.nx + 1) + (unsigned)i;
    o.f0 = p.flux[f];
    o.f1 = p.flux[f + 1];
    o.init = p.state_init[o.c];
    return true;
}
__device__ __forceinline__ void mw_finish(const gp_miniweather_params &p, const MwOperands<GP_MW_UPDATE_X> &o) {
#pragma clang fp contract(off)
    const float tend = mw_div(-(o.f1 - o.f0), p.dx, 1.0f / p.dx);
    p.state_out[o.c] = o.init + p.dt * tend;
}

__device__ __forceinline__ bool mw_load(const gp_miniweather_params &p, const MwCursor &cur, MwOperands<GP_MW_UPDATE_Z> &o) {
    int ll, k, i;
    if (!mw_update_cell(p, cur, ll, k, i)) return false;
    o.ll = ll;
    const unsigned srow = (unsigned)(p.nx + 2 * MW_HS), frow = (unsigned)(p.nx + 1);
    o.c = (unsigned)(ll * (p.nz + 2 * MW_HS) + k + MW_HS) * srow + (unsigned)(i + MW_HS);
    const unsigned f = (unsigned)(ll * (p.nz + 1) + k) * frow + (unsigned)i;
    o.f0 = p.flux[f];
    o.f1 = p.flux[f + frow];
    o.init = p.state_init[o.c];
    o.d0 = o.d1 = o.dinit = 0.f;
    if (ll == MW_WMOM) {
        // Gravity acts on the density of the forcing state.  When the forcing state is also the
        // output (second Runge-Kutta stage) other lanes overwrite that density in this very
        // kernel; in element order the density ids come first, so the value defined for this read
        // is the UPDATED one, which is recomputed from operands the kernel never writes instead
        // of being read while it changes.
        const unsigned cd = (unsigned)(k + MW_HS) * srow + (unsigned)(i + MW_HS), fd = (unsigned)k * frow + (unsigned)i;  // field 0
        if (p.state == p.state_out) {
            o.d0 = p.flux[fd];
            o.d1 = p.flux[fd + frow];
            o.dinit = p.state_init[cd];
        } else {
            o.dinit = p.state[cd];
        }
    }
    return true;
}
__device__ __forceinline__ void mw_finish(const gp_miniweather_params &p, const MwOperands<GP_MW_UPDATE_Z> &o) {
#pragma clang fp contract(off)
    const float dz_inv = 1.0f / p.dz;
    float tend = mw_div(-(o.f1 - o.f0), p.dz, dz_inv);
    if (o.ll == MW_WMOM) {
        float dens = o.dinit;
        if (p.state == p.state_out) {
            const float td = mw_div(-(o.d1 - o.d0), p.dz, dz_inv);
            dens = o.dinit + p.dt * td;
        }
        tend = tend - dens * MW_GRAV;
    }
    p.state_out[o.c] = o.init + p.dt * tend;
}

// 1 / a in fp64: the hardware's estimate (2^-23) and two Newton steps, which leaves an error of the last bit or two.
// (The compiler's own a / b is correctly rounded and handles zeros, infinities and denormals: 15 instructions with the
// scaling and the fix-up; the densities divided by here are ordinary numbers, and the quotient goes into a flux that is
// stored in fp32.)
__device__ __forceinline__ double mw_rcp(double a) {
    double y = __builtin_amdgcn_rcp(a);
    double e = __builtin_fma(-a, y, 1.0);
    y = __builtin_fma(y, e, y);
    e = __builtin_fma(-a, y, 1.0);
    return __builtin_fma(y, e, y);
}
// x^g in fp64 for an ordinary positive x (the flux kernels raise rho*theta, about 10^4-10^5, to gamma): the
// library's pow, or its exp(g log(x)), spend two thirds of their 110 instructions on arguments that cannot occur here
// and on the last bits of a result that is rounded to fp32 when the flux is stored.  This one is 45 instructions and
// good to 10^-14: x = 2^e m with m in [sqrt(1/2), sqrt(2)), log m = 2 atanh(s) with s = (m - 1) / (m + 1)
// (|s| < 0.172: the series to s^17), exp by n = round(y / ln 2) and the Taylor series of the rest to the 12th power.
__device__ __forceinline__ double mw_pow_pos(double x, double g) {
    double m = __builtin_amdgcn_frexp_mant(x);  // [1/2, 1)
    int e = __builtin_amdgcn_frexp_exp(x);
    if (m < 0.70710678118654752440) { m *= 2.0; e -= 1; }
    const double s = (m - 1.0) * mw_rcp(m + 1.0), s2 = s * s;
    double a = 1.0 / 17.0;
    a = __builtin_fma(a, s2, 1.0 / 15.0);
    a = __builtin_fma(a, s2, 1.0 / 13.0);
    a = __builtin_fma(a, s2, 1.0 / 11.0);
    a = __builtin_fma(a, s2, 1.0 / 9.0);
    a = __builtin_fma(a, s2, 1.0 / 7.0);
    a = __builtin_fma(a, s2, 1.0 / 5.0);
    a = __builtin_fma(a, s2, 1.0 / 3.0);
    a = __builtin_fma(a, s2, 1.0);
    const double ln_x = __builtin_fma((double)e, 0.69314718055994530942, (s + s) * a);
    const double y = g * ln_x;
    const double n = __builtin_rint(y * 1.44269504088896340736);
    double r = __builtin_fma(-n, 0.693147180369123816490, y);  // ln 2 in two pieces: n * the first is exact
    r = __builtin_fma(-n, 1.90821492927058770002e-10, r);
    double q = 1.0 / 479001600.0;
    q = __builtin_fma(q, r, 1.0 / 39916800.0);
    q = __builtin_fma(q, r, 1.0 / 3628800.0);
    q = __builtin_fma(q, r, 1.0 / 362880.0);
    q = __builtin_fma(q, r, 1.0 / 40320.0);
    q = __builtin_fma(q, r, 1.0 / 5040.0);
    q = __builtin_fma(q, r, 1.0 / 720.0);
    q = __builtin_fma(q, r, 1.0 / 120.0);
    q = __builtin_fma(q, r, 1.0 / 24.0);
    q = __builtin_fma(q, r, 1.0 / 6.0);
    q = __builtin_fma(q, r, 0.5);
    q = __builtin_fma(q, r, 1.0);
    q = __builtin_fma(q, r, 1.0);
    return __builtin_amdgcn_ldexp(q, (int)n);
}

__device__ __forceinline__ bool mw_load(const gp_miniweather_params &p, const MwCursor &cur, MwOperands<GP_MW_FLUX_X> &o) {
    const MwHydro hy(p.hydro, p.nz);
    cur.lane(o.k, o.i);
    if (o.k >= p.nz) return false;
    // (32-bit offsets from the base: the four fields together stay below 2^31 elements, gp_launch_miniweather)
    const unsigned plane = (unsigned)(p.nz + 2 * MW_HS) * (unsigned)(p.nx + 2 * MW_HS);
    const unsigned at = (unsigned)(o.k + MW_HS) * (unsigned)(p.nx + 2 * MW_HS) + (unsigned)o.i;
#pragma unroll
    for (int ll = 0; ll < MW_VARS; ++ll) {
        const float *c = p.state + (at + (unsigned)ll * plane);
#pragma unroll
        for (int s = 0; s < 4; ++s) o.s[ll][s] = c[s];
    }
    o.h0 = hy.dens_cell[o.k + MW_HS];
    o.h1 = hy.dens_theta_cell[o.k + MW_HS];
    return true;
}
// the four fluxes through one x interface from the four cell averages around it (miniweather.tr.cu:337-348)
__device__ __forceinline__ void mw_flux_x_point(const float (&s)[MW_VARS][4], float h0, float h1, float hv_coef, float (&f)[MW_VARS]) {
#pragma clang fp contract(off)
    float vals[MW_VARS], d3[MW_VARS];
#pragma unroll
    for (int ll = 0; ll < MW_VARS; ++ll) mw_reconstruct(s[ll], hv_coef, vals[ll], d3[ll]);
    const double r = vals[MW_DENS] + h0;
    // (one reciprocal for the three quotients, and a power function for arguments that occur: with the compiler's
    // divisions and exp(gamma log(.)) this kernel spent 55 us on 35 us of memory traffic; a general pow made it 80)
    const double r_inv = mw_rcp(r);
    const double u = vals[MW_UMOM] * r_inv;
    const double w = vals[MW_WMOM] * r_inv;
    const double th = (vals[MW_RHOT] + h1) * r_inv;
    const double pr = MW_C0 * mw_pow_pos(r * th, (double)MW_GAMMA);
    f[MW_DENS] = (float)(r * u - d3[MW_DENS]);
    f[MW_UMOM] = (float)(r * u * u + pr - d3[MW_UMOM]);
    f[MW_WMOM] = (float)(r * u * w - d3[MW_WMOM]);
    f[MW_RHOT] = (float)(r * u * th - d3[MW_RHOT]);
}
__device__ __forceinline__ void mw_finish(const gp_miniweather_params &p, const MwOperands<GP_MW_FLUX_X> &o) {
    const MwView v{p.nx, p.nz};
    const float hv_coef = -MW_HV_BETA * p.dx / (16 * p.dt);
    float f[MW_VARS];
    mw_flux_x_point(o.s, o.h0, o.h1, hv_coef, f);
    const unsigned plane = (unsigned)(p.nz + 1) * (unsigned)(p.nx + 1), at = (unsigned)o.k * (unsigned)(p.nx + 1) + (unsigned)o.i;
#pragma unroll
    for (int ll = 0; ll < MW_VARS; ++ll) p.flux[at + (unsigned)ll * plane] = f[ll];
}

__device__ __forceinline__ bool mw_load(const gp_miniweather_params &p, const MwCursor &cur, MwOperands<GP_MW_FLUX_Z> &o) {
    const MwHydro hy(p.hydro, p.nz);
    cur.lane(o.k, o.i);
    if (o.k >= p.nz + 1) return false;
    const unsigned row = (unsigned)(p.nx + 2 * MW_HS), plane = (unsigned)(p.nz + 2 * MW_HS) * row;
    const unsigned at = (unsigned)o.k * row + (unsigned)(o.i + MW_HS);
#pragma unroll
    for (int ll = 0; ll < MW_VARS; ++ll) {
        const float *c = p.state + (at + (unsigned)ll * plane);
#pragma unroll
        for (int s = 0; s < 4; ++s) o.s[ll][s] = c[(unsigned)s * row];
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
    // (the power through the fp64 routine above, rounded to fp32 once: nearer to the exact power than powf is, and cheaper
    // than the library's powf, which carries its logarithm in two floats: 4-7 us per launch at 3200 x 1600)
    const float pr = MW_C0 * (float)mw_pow_pos((double)(r * th), (double)MW_GAMMA) - o.h2;
    if (o.k == 0 || o.k == p.nz) {  // no flow through the bottom and top faces, exact mass conservation
        w = 0.f;
        d3[MW_DENS] = 0.f;
    }
    const unsigned plane = (unsigned)(p.nz + 1) * (unsigned)(p.nx + 1), at = (unsigned)o.k * (unsigned)(p.nx + 1) + (unsigned)o.i;
    p.flux[at + MW_DENS * plane] = r * w - d3[MW_DENS];
    p.flux[at + MW_UMOM * plane] = r * w * u - d3[MW_UMOM];
    p.flux[at + MW_WMOM * plane] = r * w * w + pr - d3[MW_WMOM];
    p.flux[at + MW_RHOT * plane] = r * w * th - d3[MW_RHOT];
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
#ifndef GP_MW_FLUX_U
#define GP_MW_FLUX_U 1  // (measured 2 and 3: 3 and 8 % slower per execute; the flux kernels are bound by the instructions they issue)
#endif
        constexpr bool FLUX = KIND == GP_MW_FLUX_X || KIND == GP_MW_FLUX_Z;
        constexpr int U = FLUX ? GP_MW_FLUX_U : 4;
        MwCursor cur((unsigned)first * MW_TILE, KIND == GP_MW_FLUX_X ? (unsigned)p.nx + 1 : (unsigned)p.nx);
        for (int t = first; t < last; t += U) {
            MwOperands<KIND> op[U];
            bool ok[U];
#pragma unroll
            for (int j = 0; j < U; ++j) {
                ok[j] = t + j < last && mw_load(p, cur, op[j]);
                cur.next_tile();
            }
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
