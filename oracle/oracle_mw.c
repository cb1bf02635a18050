/* TEST INFRASTRUCTURE ONLY: CPU restatement of the reference's miniWeather workload, used by
 * tests/ and by smoke/bench checkers; no product code may call it.
 *
 * Follows reference src/workloads/miniweather.tr.cu (the block-level-preemptible build of the
 * stratified-flow mini-app): constants :22-61, time step :184-206, the three kernels of a
 * semi-discrete step :216-276, kernel bodies :318-349 (x flux), :381-393 (x update), :429-468
 * (z flux), :485-502 (z update), :510-520 (x halo), :530-552 (z halo), initial state :555-686,
 * analytic profiles :689-775, reductions :906-932.
 *
 * Arithmetic types are the reference's: the state is fp32, the x flux is formed in fp64, the z
 * flux in fp32.  The reference is C++: a math call whose arguments are all float resolves to the
 * float overload there, so this C file names powf / expf / sqrtf / cosf in exactly those places.
 * A "tile" is 256 consecutive element ids of a kernel (the reference's thread
 * block), processed in increasing id order.
 *
 * One reference quirk is settled deliberately: in the second Runge-Kutta stage of a z sweep the
 * forcing state and the output state are the same array, and the vertical-momentum update reads
 * the density of the forcing state while other threads overwrite it (:493-496).  Executed in id
 * order (density ids precede momentum ids) the read sees the UPDATED density; that order is what
 * this restatement defines, and what the device code reproduces without depending on timing.
 *
 * Pinned by tests/test_oracle_miniweather.py: hydrostatic rest state stays at rest, mass is
 * conserved to rounding, x-translation and mirror symmetry, cubic-exact interface interpolation,
 * initial hydrostatic column against the closed-form Exner profile, and resume-from-any-kernel
 * equals the uninterrupted step.  The reference holds no golden output for this workload. */
#include <math.h>
#include <stdlib.h>
#include <string.h>

typedef float real;

static const real pi = 3.14159265358979323846264338327;
static const real grav = 9.8;
static const real cp = 1004.;
static const real cv = 717.;
static const real rd = 287.;
static const real p0 = 1.e5;
static const real C0 = 27.5629410929725921310572974482;
static const real gamm = 1.40027894002789400278940027894;
static const real xlen = 2.e4;
static const real zlen = 1.e4;
static const real hv_beta = 0.05;
static const real cfl = 1.50;
static const real max_speed = 450;
enum { HS = 2, NUM_VARS = 4, ID_DENS = 0, ID_UMOM = 1, ID_WMOM = 2, ID_RHOT = 3 };
enum { K_HALO_X = 0, K_FLUX_X = 1, K_UPDATE_X = 2, K_HALO_Z = 3, K_FLUX_Z = 4, K_UPDATE_Z = 5 };
enum { TILE = 256 };

/* hydrostatic arrays share one buffer: cell density (nz+4), cell density*theta (nz+4), interface
 * density (nz+1), interface density*theta (nz+1), interface pressure (nz+1), 4 boundary ratios */
long mw_hydro_elems(int nz) { return 2L * (nz + 2 * HS) + 3L * (nz + 1) + 4; }
long mw_state_elems(int nx, int nz) { return (long)NUM_VARS * (nz + 2 * HS) * (nx + 2 * HS); }
long mw_flux_elems(int nx, int nz) { return (long)NUM_VARS * (nz + 1) * (nx + 1); }

typedef struct {
    const real *dens_cell, *dens_theta_cell, *dens_int, *dens_theta_int, *pressure_int, *cell_const;
} Hydro;
static Hydro hydro_view(const real *h, int nz) {
    Hydro v;
    v.dens_cell = h;
    v.dens_theta_cell = v.dens_cell + nz + 2 * HS;
    v.dens_int = v.dens_theta_cell + nz + 2 * HS;
    v.dens_theta_int = v.dens_int + nz + 1;
    v.pressure_int = v.dens_theta_int + nz + 1;
    v.cell_const = v.pressure_int + nz + 1;
    return v;
}

real mw_dx(int nx) { return xlen / nx; }
real mw_dz(int nz) { return zlen / nz; }
real mw_dt(int nx, int nz) {
    real dx = mw_dx(nx), dz = mw_dz(nz);
    return (dx < dz ? dx : dz) / max_speed * cfl; /* :584 */
}

/* number of element ids of a kernel; the z halo covers (nx+4)*4 ids (the reference's launch
 * arithmetic at :252 loses a pair of parentheses and covers fewer) */
long mw_kernel_ids(int kernel, int nx, int nz) {
    switch (kernel) {
        case K_HALO_X: return (long)nz * NUM_VARS;
        case K_FLUX_X: return (long)nz * (nx + 1);
        case K_UPDATE_X: return (long)nz * nx * NUM_VARS;
        case K_HALO_Z: return (long)(nx + 2 * HS) * NUM_VARS;
        case K_FLUX_Z: return (long)nx * (nz + 1);
        case K_UPDATE_Z: return (long)nx * nz * NUM_VARS;
    }
    return 0;
}
long mw_kernel_tiles(int kernel, int nx, int nz) { return (mw_kernel_ids(kernel, nx, nz) + TILE - 1) / TILE; }

#define ST(ll, kk, ii) ((long)(ll) * (nz + 2 * HS) * (nx + 2 * HS) + (long)(kk) * (nx + 2 * HS) + (ii))
#define FX(ll, kk, ii) ((long)(ll) * (nz + 1) * (nx + 1) + (long)(kk) * (nx + 1) + (ii))

static void one_id(int kernel, long id, int nx, int nz, real dt, real *state, real *flux, const real *state_init,
                   real *state_out, const Hydro *hy) {
    const real dx = mw_dx(nx), dz = mw_dz(nz);
    switch (kernel) {
        case K_HALO_X: { /* :510-520, periodic in x */
            int ll = (int)(id / nz), k = (int)(id % nz);
            if (ll < NUM_VARS) {
                state[ST(ll, k + HS, 0)] = state[ST(ll, k + HS, nx + HS - 2)];
                state[ST(ll, k + HS, 1)] = state[ST(ll, k + HS, nx + HS - 1)];
                state[ST(ll, k + HS, nx + HS)] = state[ST(ll, k + HS, HS)];
                state[ST(ll, k + HS, nx + HS + 1)] = state[ST(ll, k + HS, HS + 1)];
            }
            break;
        }
        case K_FLUX_X: { /* :318-349 */
            int k = (int)(id / (nx + 1)), i = (int)(id % (nx + 1));
            if (k < nz) {
                real stencil[4], d3_vals[NUM_VARS], vals[NUM_VARS];
                real hv_coef = -hv_beta * dx / (16 * dt);
                for (int ll = 0; ll < NUM_VARS; ll++) {
                    for (int s = 0; s < 4; s++) stencil[s] = state[ST(ll, k + HS, i + s)];
                    vals[ll] = (-stencil[0] + 7 * (stencil[1] + stencil[2]) - stencil[3]) / 12;
                    d3_vals[ll] = (-stencil[0] + 3 * (stencil[1] - stencil[2]) + stencil[3]) * hv_coef;
                }
                double r = vals[ID_DENS] + hy->dens_cell[k + HS];
                double u = vals[ID_UMOM] / r;
                double w = vals[ID_WMOM] / r;
                double t = (vals[ID_RHOT] + hy->dens_theta_cell[k + HS]) / r;
                double p = C0 * pow((r * t), gamm);
                flux[FX(ID_DENS, k, i)] = r * u - d3_vals[ID_DENS];
                flux[FX(ID_UMOM, k, i)] = r * u * u + p - d3_vals[ID_UMOM];
                flux[FX(ID_WMOM, k, i)] = r * u * w - d3_vals[ID_WMOM];
                flux[FX(ID_RHOT, k, i)] = r * u * t - d3_vals[ID_RHOT];
            }
            break;
        }
        case K_UPDATE_X: { /* :381-393 */
            int k = (int)((id / nx) % nz), i = (int)(id % nx), ll = (int)(id / nx / nz);
            if (ll < NUM_VARS) {
                real tend = -(flux[FX(ll, k, i + 1)] - flux[FX(ll, k, i)]) / dx;
                state_out[ST(ll, k + HS, i + HS)] = state_init[ST(ll, k + HS, i + HS)] + dt * tend;
            }
            break;
        }
        case K_HALO_Z: { /* :530-552 */
            int i = (int)(id % (nx + 2 * HS)), ll = (int)(id / (nx + 2 * HS));
            if (ll < NUM_VARS) {
                if (ll == ID_WMOM) {
                    state[ST(ll, 0, i)] = 0.;
                    state[ST(ll, 1, i)] = 0.;
                    state[ST(ll, nz + HS, i)] = 0.;
                    state[ST(ll, nz + HS + 1, i)] = 0.;
                } else if (ll == ID_UMOM) {
                    state[ST(ll, 0, i)] = state[ST(ll, HS, i)] * hy->cell_const[0];
                    state[ST(ll, 1, i)] = state[ST(ll, HS, i)] * hy->cell_const[1];
                    state[ST(ll, nz + HS, i)] = state[ST(ll, nz + HS - 1, i)] * hy->cell_const[2];
                    state[ST(ll, nz + HS + 1, i)] = state[ST(ll, nz + HS - 1, i)] * hy->cell_const[3];
                } else {
                    state[ST(ll, 0, i)] = state[ST(ll, HS, i)];
                    state[ST(ll, 1, i)] = state[ST(ll, HS, i)];
                    state[ST(ll, nz + HS, i)] = state[ST(ll, nz + HS - 1, i)];
                    state[ST(ll, nz + HS + 1, i)] = state[ST(ll, nz + HS - 1, i)];
                }
            }
            break;
        }
        case K_FLUX_Z: { /* :429-468 */
            int i = (int)(id % nx), k = (int)(id / nx);
            if (k < nz + 1) {
                real r, u, w, t, p, stencil[4], d3_vals[NUM_VARS], vals[NUM_VARS], hv_coef;
                hv_coef = -hv_beta * dz / (16 * dt);
                for (int ll = 0; ll < NUM_VARS; ll++) {
                    for (int s = 0; s < 4; s++) stencil[s] = state[ST(ll, k + s, i + HS)];
                    vals[ll] = (-stencil[0] + 7 * (stencil[1] + stencil[2]) - stencil[3]) / 12;
                    d3_vals[ll] = (-stencil[0] + 3 * (stencil[1] - stencil[2]) + stencil[3]) * hv_coef;
                }
                r = vals[ID_DENS] + hy->dens_int[k];
                u = vals[ID_UMOM] / r;
                w = vals[ID_WMOM] / r;
                t = (vals[ID_RHOT] + hy->dens_theta_int[k]) / r;
                p = C0 * powf((r * t), gamm) - hy->pressure_int[k];
                if (k == 0 || k == nz) {
                    w = 0;
                    d3_vals[ID_DENS] = 0;
                }
                flux[FX(ID_DENS, k, i)] = r * w - d3_vals[ID_DENS];
                flux[FX(ID_UMOM, k, i)] = r * w * u - d3_vals[ID_UMOM];
                flux[FX(ID_WMOM, k, i)] = r * w * w + p - d3_vals[ID_WMOM];
                flux[FX(ID_RHOT, k, i)] = r * w * t - d3_vals[ID_RHOT];
            }
            break;
        }
        case K_UPDATE_Z: { /* :485-502 */
            int i = (int)(id % nx), k = (int)((id / nx) % nz), ll = (int)(id / nx / nz);
            if (ll < NUM_VARS) {
                real tend = -(flux[FX(ll, k + 1, i)] - flux[FX(ll, k, i)]) / dz;
                if (ll == ID_WMOM) tend = tend - state[ST(ID_DENS, k + HS, i + HS)] * grav;
                state_out[ST(ll, k + HS, i + HS)] = state_init[ST(ll, k + HS, i + HS)] + dt * tend;
            }
            break;
        }
    }
}

/* Runs tile `tile` (ids tile*256 .. tile*256+255, clipped) of one kernel. */
void mw_run_tile(int kernel, long tile, int nx, int nz, real dt, real *state, real *flux, const real *state_init,
                 real *state_out, const real *hydro) {
    Hydro hy = hydro_view(hydro, nz);
    long n = mw_kernel_ids(kernel, nx, nz);
    long lo = tile * TILE, hi = lo + TILE < n ? lo + TILE : n;
    for (long id = lo; id < hi; ++id) one_id(kernel, id, nx, nz, dt, state, flux, state_init, state_out, &hy);
}

/* Kernel `kid` (0..35) of a time step: semi-discrete step kid/3, kernel kid%3 of it.
 * Step table :190-204: sweeps X, Z, Z, X; each sweep runs the three Runge-Kutta stages
 * (init, forcing, out, dt divisor) = (s, s, t, 3), (s, t, t, 2), (s, t, s, 1). */
void mw_kernel_operands(int kid, real *state, real *state_tmp, real dt, int *kernel, real **forcing, const real **init,
                        real **out, real *dt_stage) {
    int step = kid / 3, sub = kid % 3, sweep = step / 3, stage = step % 3;
    int dir_z = (sweep == 1 || sweep == 2);
    *kernel = (dir_z ? 3 : 0) + sub;
    *init = state;
    *forcing = stage == 0 ? state : state_tmp;
    *out = stage == 2 ? state : state_tmp;
    *dt_stage = stage == 0 ? dt / 3 : stage == 1 ? dt / 2 : dt / 1;
}

/* Runs tiles [tile_lo, tile_hi) of kernel kid (tile_hi < 0: to the end). */
void mw_run_kernel(int kid, long tile_lo, long tile_hi, int nx, int nz, real dt, real *state, real *state_tmp,
                   real *flux, const real *hydro) {
    int kernel;
    real *forcing, *out, dts;
    const real *init;
    mw_kernel_operands(kid, state, state_tmp, dt, &kernel, &forcing, &init, &out, &dts);
    long nt = mw_kernel_tiles(kernel, nx, nz);
    if (tile_hi < 0 || tile_hi > nt) tile_hi = nt;
    for (long t = tile_lo; t < tile_hi; ++t) mw_run_tile(kernel, t, nx, nz, dts, forcing, flux, init, out, hydro);
}

/* perform_timestep(..., start_from) :184-206: kernels start_from .. 35. */
void mw_timestep(int nx, int nz, real dt, real *state, real *state_tmp, real *flux, const real *hydro, int start_from) {
    for (int kid = start_from; kid < 36; ++kid) mw_run_kernel(kid, 0, -1, nx, nz, dt, state, state_tmp, flux, hydro);
}

/* ---- initial state ----------------------------------------------------------------------- */
static void hydro_const_theta(real z, real *r, real *t) { /* :744-753 */
    const real theta0 = 300., exner0 = 1.;
    real p, exner, rt;
    *t = theta0;
    exner = exner0 - grav * z / (cp * theta0);
    p = p0 * powf(exner, (cp / rd));   /* all-float arguments: the C++ overload the reference compiles to */
    rt = pow((p / C0), (1. / gamm));   /* a double exponent: double pow */
    *r = rt / *t;
}
static void hydro_const_bvfreq(real z, real bv_freq0, real *r, real *t) { /* :756-765 */
    const real theta0 = 300., exner0 = 1.;
    real p, exner, rt;
    *t = theta0 * expf(bv_freq0 * bv_freq0 / grav * z);
    exner = exner0 - grav * grav / (cp * bv_freq0 * bv_freq0) * (*t - theta0) / (*t * theta0);
    p = p0 * powf(exner, (cp / rd));
    rt = pow((p / C0), (1. / gamm));
    *r = rt / *t;
}
static real sample_ellipse_cosine(real x, real z, real amp, real x0, real z0, real xrad, real zrad) { /* :768-775 */
    real dist = sqrtf(((x - x0) / xrad) * ((x - x0) / xrad) + ((z - z0) / zrad) * ((z - z0) / zrad)) * pi / 2.;
    if (dist <= pi / 2.) return amp * pow(cosf(dist), 2.);
    return 0.;
}
/* data_spec: 1 collision, 2 thermal, 3 gravity waves, 5 density current, 6 injection (:689-741) */
static void profile(int spec, real x, real z, real *r, real *u, real *w, real *t, real *hr, real *ht) {
    *r = 0.; *t = 0.; *u = 0.; *w = 0.;
    if (spec == 3) { hydro_const_bvfreq(z, 0.02, hr, ht); *u = 15.; return; }
    hydro_const_theta(z, hr, ht);
    if (spec == 1) {
        *t = *t + sample_ellipse_cosine(x, z, 20., xlen / 2, 2000., 2000., 2000.);
        *t = *t + sample_ellipse_cosine(x, z, -20., xlen / 2, 8000., 2000., 2000.);
    } else if (spec == 2) {
        *t = *t + sample_ellipse_cosine(x, z, 3., xlen / 2, 2000., 2000., 2000.);
    } else if (spec == 5) {
        *t = *t + sample_ellipse_cosine(x, z, -20., xlen / 2, 5000., 4000., 2000.);
    }
}

/* sci_init :555-686: 3x3 Gauss-Legendre cell averages of the perturbation, hydrostatic columns. */
void mw_init(int nx, int nz, int spec, real *state, real *hydro) {
    static const real qpoints[] = {0.112701665379258311482073460022E0, 0.500000000000000000000000000000E0, 0.887298334620741688517926539980E0};
    static const real qweights[] = {0.277777777777777777777777777779E0, 0.444444444444444444444444444444E0, 0.277777777777777777777777777779E0};
    const real dx = mw_dx(nx), dz = mw_dz(nz);
    real x, z, r, u, w, t, hr, ht;
    real *hy_dens_cell = hydro, *hy_dens_theta_cell = hy_dens_cell + nz + 2 * HS, *hy_dens_int = hy_dens_theta_cell + nz + 2 * HS,
         *hy_dens_theta_int = hy_dens_int + nz + 1, *hy_pressure_int = hy_dens_theta_int + nz + 1, *cell_const = hy_pressure_int + nz + 1;
    for (int k = 0; k < nz + 2 * HS; k++) {
        for (int i = 0; i < nx + 2 * HS; i++) {
            for (int ll = 0; ll < NUM_VARS; ll++) state[ST(ll, k, i)] = 0.;
            for (int kk = 0; kk < 3; kk++) {
                for (int ii = 0; ii < 3; ii++) {
                    x = (0 + i - HS + 0.5) * dx + (qpoints[ii] - 0.5) * dx;
                    z = (0 + k - HS + 0.5) * dz + (qpoints[kk] - 0.5) * dz;
                    profile(spec, x, z, &r, &u, &w, &t, &hr, &ht);
                    state[ST(ID_DENS, k, i)] = state[ST(ID_DENS, k, i)] + r * qweights[ii] * qweights[kk];
                    state[ST(ID_UMOM, k, i)] = state[ST(ID_UMOM, k, i)] + (r + hr) * u * qweights[ii] * qweights[kk];
                    state[ST(ID_WMOM, k, i)] = state[ST(ID_WMOM, k, i)] + (r + hr) * w * qweights[ii] * qweights[kk];
                    state[ST(ID_RHOT, k, i)] = state[ST(ID_RHOT, k, i)] + ((r + hr) * (t + ht) - hr * ht) * qweights[ii] * qweights[kk];
                }
            }
        }
    }
    for (int k = 0; k < nz + 2 * HS; k++) {
        hy_dens_cell[k] = 0.;
        hy_dens_theta_cell[k] = 0.;
        for (int kk = 0; kk < 3; kk++) {
            z = (0 + k - HS + 0.5) * dz; /* the reference samples the cell centre three times (:625-626) */
            profile(spec, 0., z, &r, &u, &w, &t, &hr, &ht);
            hy_dens_cell[k] = hy_dens_cell[k] + hr * qweights[kk];
            hy_dens_theta_cell[k] = hy_dens_theta_cell[k] + hr * ht * qweights[kk];
        }
    }
    for (int k = 0; k < nz + 1; k++) {
        z = (0 + k) * dz;
        profile(spec, 0., z, &r, &u, &w, &t, &hr, &ht);
        hy_dens_int[k] = hr;
        hy_dens_theta_int[k] = hr * ht;
        hy_pressure_int[k] = C0 * powf((hr * ht), gamm);
    }
    cell_const[0] = hy_dens_cell[0] / hy_dens_cell[HS]; /* :679-683 */
    cell_const[1] = hy_dens_cell[1] / hy_dens_cell[HS];
    cell_const[2] = hy_dens_cell[nz + HS] / hy_dens_cell[nz + HS - 1];
    cell_const[3] = hy_dens_cell[nz + HS + 1] / hy_dens_cell[nz + HS - 1];
}

/* reductions :906-932: domain mass and total energy in fp64. */
void mw_reductions(int nx, int nz, const real *state, const real *hydro, double *mass_out, double *te_out) {
    Hydro hy = hydro_view(hydro, nz);
    const real dx = mw_dx(nx), dz = mw_dz(nz);
    double mass = 0, te = 0;
    for (int k = 0; k < nz; k++) {
        for (int i = 0; i < nx; i++) {
            double r = state[ST(ID_DENS, k + HS, i + HS)] + hy.dens_cell[HS + k];
            double u = state[ST(ID_UMOM, k + HS, i + HS)] / r;
            double w = state[ST(ID_WMOM, k + HS, i + HS)] / r;
            double th = (state[ST(ID_RHOT, k + HS, i + HS)] + hy.dens_theta_cell[HS + k]) / r;
            double p = C0 * pow(r * th, gamm);
            double t = th / pow(p0 / p, rd / cp);
            double ke = r * (u * u + w * w);
            double ie = r * cv * t;
            mass += r * dx * dz;
            te += (ke + ie) * dx * dz;
        }
    }
    *mass_out = mass;
    *te_out = te;
}
