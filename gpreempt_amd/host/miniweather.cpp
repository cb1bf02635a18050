// Host side of the miniWeather workload: initial state and conservation diagnostics
// (reference src/workloads/miniweather.tr.cu:555-686, :689-775, :906-932).  The arithmetic keeps
// the reference's mix of fp32 variables and fp64 library calls.
#include "workloads/scicomput.h"
#include <algorithm>
#include <cmath>

namespace SciCompute {

namespace {
typedef float real;
const real kPi = 3.14159265358979323846264338327, kGrav = 9.8, kCp = 1004., kCv = 717., kRd = 287., kP0 = 1.e5;
const real kC0 = 27.5629410929725921310572974482, kGamma = 1.40027894002789400278940027894;
const real kXlen = 2.e4, kZlen = 1.e4, kMaxSpeed = 450, kCfl = 1.50;
const real kTheta0 = 300., kExner0 = 1.;
const real kQPoints[3] = {0.112701665379258311482073460022E0, 0.500000000000000000000000000000E0, 0.887298334620741688517926539980E0};
const real kQWeights[3] = {0.277777777777777777777777777779E0, 0.444444444444444444444444444444E0, 0.277777777777777777777777777779E0};

struct Column { real hr, ht; };      // hydrostatic density and potential temperature at a height
struct Sample { real r, u, w, t; Column bg; };

// density from pressure through the equation of state p = C0 (rho theta)^gamma
real density_from_exner(real exner, real theta) {
    real p = kP0 * std::pow(exner, (kCp / kRd));
    real rt = std::pow((p / kC0), (1. / kGamma));
    return rt / theta;
}
Column const_theta_column(real z) {  // :744-753
    real exner = kExner0 - kGrav * z / (kCp * kTheta0);
    return Column{density_from_exner(exner, kTheta0), kTheta0};
}
Column const_bvfreq_column(real z, real bv) {  // :756-765
    real t = kTheta0 * std::exp(bv * bv / kGrav * z);
    real exner = kExner0 - kGrav * kGrav / (kCp * bv * bv) * (t - kTheta0) / (t * kTheta0);
    return Column{density_from_exner(exner, t), t};
}
real cosine_bump(real x, real z, real amp, real x0, real z0, real xrad, real zrad) {  // :768-775
    real dist = std::sqrt(((x - x0) / xrad) * ((x - x0) / xrad) + ((z - z0) / zrad) * ((z - z0) / zrad)) * kPi / 2.;
    if (dist <= kPi / 2.) return amp * std::pow(std::cos(dist), 2.);
    return 0.;
}
Sample sample_at(int spec, real x, real z) {  // :689-741
    Sample s{0.f, 0.f, 0.f, 0.f, Column{0.f, 0.f}};
    if (spec == GravityWaves) {
        s.bg = const_bvfreq_column(z, 0.02);
        s.u = 15.;
        return s;
    }
    s.bg = const_theta_column(z);
    switch (spec) {
        case Collision:
            s.t = s.t + cosine_bump(x, z, 20., kXlen / 2, 2000., 2000., 2000.);
            s.t = s.t + cosine_bump(x, z, -20., kXlen / 2, 8000., 2000., 2000.);
            break;
        case Thermal: s.t = s.t + cosine_bump(x, z, 3., kXlen / 2, 2000., 2000., 2000.); break;
        case DensityCurrent: s.t = s.t + cosine_bump(x, z, -20., kXlen / 2, 5000., 4000., 2000.); break;
        default: break;  // Injection: background only
    }
    return s;
}
}  // namespace

Grid make_grid(int nx, int nz) {
    Grid g;
    g.nx = nx; g.nz = nz;
    g.dx = kXlen / nx;
    g.dz = kZlen / nz;
    g.dt = std::min(g.dx, g.dz) / kMaxSpeed * kCfl;
    return g;
}

void initial_state(const Grid &g, int spec, std::vector<float> &state, std::vector<float> &hydro) {
    const int nx = g.nx, nz = g.nz, W = nx + 4, H = nz + 4;
    const real dx = g.dx, dz = g.dz;
    state.assign(state_elems(g), 0.f);
    hydro.assign(hydro_elems(g), 0.f);
    real *dens = state.data(), *umom = dens + (size_t)H * W, *wmom = umom + (size_t)H * W, *rhot = wmom + (size_t)H * W;
    for (int k = 0; k < H; ++k) {
        for (int i = 0; i < W; ++i) {
            const size_t c = (size_t)k * W + i;
            for (int kk = 0; kk < 3; ++kk) {
                for (int ii = 0; ii < 3; ++ii) {
                    real x = (0 + i - 2 + 0.5) * dx + (kQPoints[ii] - 0.5) * dx;
                    real z = (0 + k - 2 + 0.5) * dz + (kQPoints[kk] - 0.5) * dz;
                    const Sample s = sample_at(spec, x, z);
                    const real r = s.r, u = s.u, w = s.w, t = s.t, hr = s.bg.hr, ht = s.bg.ht;
                    dens[c] = dens[c] + r * kQWeights[ii] * kQWeights[kk];
                    umom[c] = umom[c] + (r + hr) * u * kQWeights[ii] * kQWeights[kk];
                    wmom[c] = wmom[c] + (r + hr) * w * kQWeights[ii] * kQWeights[kk];
                    rhot[c] = rhot[c] + ((r + hr) * (t + ht) - hr * ht) * kQWeights[ii] * kQWeights[kk];
                }
            }
        }
    }
    real *cell_dens = hydro.data(), *cell_dens_theta = cell_dens + H, *int_dens = cell_dens_theta + H;
    real *int_dens_theta = int_dens + nz + 1, *int_pressure = int_dens_theta + nz + 1, *ratios = int_pressure + nz + 1;
    for (int k = 0; k < H; ++k) {
        // the reference evaluates the cell centre once per quadrature weight (:625-634)
        for (int kk = 0; kk < 3; ++kk) {
            real z = (0 + k - 2 + 0.5) * dz;
            const Column bg = sample_at(spec, 0., z).bg;
            cell_dens[k] = cell_dens[k] + bg.hr * kQWeights[kk];
            cell_dens_theta[k] = cell_dens_theta[k] + bg.hr * bg.ht * kQWeights[kk];
        }
    }
    for (int k = 0; k < nz + 1; ++k) {
        real z = (0 + k) * dz;
        const Column bg = sample_at(spec, 0., z).bg;
        int_dens[k] = bg.hr;
        int_dens_theta[k] = bg.hr * bg.ht;
        int_pressure[k] = kC0 * std::pow((bg.hr * bg.ht), kGamma);
    }
    ratios[0] = cell_dens[0] / cell_dens[2];  // :679-683
    ratios[1] = cell_dens[1] / cell_dens[2];
    ratios[2] = cell_dens[nz + 2] / cell_dens[nz + 1];
    ratios[3] = cell_dens[nz + 3] / cell_dens[nz + 1];
}

void reductions(const Grid &g, const float *state, const float *hydro, double &mass, double &te) {
    const int nx = g.nx, nz = g.nz, W = nx + 4, H = nz + 4;
    const float *dens = state, *umom = dens + (size_t)H * W, *wmom = umom + (size_t)H * W, *rhot = wmom + (size_t)H * W;
    const float *cell_dens = hydro, *cell_dens_theta = hydro + H;
    mass = 0;
    te = 0;
    for (int k = 0; k < nz; ++k) {
        for (int i = 0; i < nx; ++i) {
            const size_t c = (size_t)(k + 2) * W + i + 2;
            double r = dens[c] + cell_dens[2 + k];
            double u = umom[c] / r;
            double w = wmom[c] / r;
            double th = (rhot[c] + cell_dens_theta[2 + k]) / r;
            double p = kC0 * std::pow(r * th, kGamma);
            double t = th / std::pow(kP0 / p, kRd / kCp);
            double ke = r * (u * u + w * w);
            double ie = r * kCv * t;
            mass += r * g.dx * g.dz;
            te += (ke + ie) * g.dx * g.dz;
        }
    }
}

}  // namespace SciCompute
