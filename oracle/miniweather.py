"""numpy front end of the miniWeather oracle (oracle_mw.c).

TEST INFRASTRUCTURE ONLY: imported by tests/ and by checkers in __graft_entry__.smoke() /
bench.py, never by the product path.
"""
import ctypes as C

import numpy as np

from . import oracle as _O

HALO_X, FLUX_X, UPDATE_X, HALO_Z, FLUX_Z, UPDATE_Z = range(6)
COLLISION, THERMAL, GRAVITY_WAVES, DENSITY_CURRENT, INJECTION = 1, 2, 3, 5, 6
KERNELS_PER_STEP = 36
HS, NUM_VARS = 2, 4
_FP = C.POINTER(C.c_float)
_ready = False


def _lib():
    global _ready
    L = _O.lib()
    if not _ready:
        for name in ("mw_hydro_elems",):
            getattr(L, name).restype = C.c_long
            getattr(L, name).argtypes = [C.c_int]
        for name in ("mw_state_elems", "mw_flux_elems"):
            getattr(L, name).restype = C.c_long
            getattr(L, name).argtypes = [C.c_int, C.c_int]
        for name in ("mw_kernel_ids", "mw_kernel_tiles"):
            getattr(L, name).restype = C.c_long
            getattr(L, name).argtypes = [C.c_int, C.c_int, C.c_int]
        L.mw_dx.restype = L.mw_dz.restype = C.c_float
        L.mw_dx.argtypes = L.mw_dz.argtypes = [C.c_int]
        L.mw_dt.restype = C.c_float
        L.mw_dt.argtypes = [C.c_int, C.c_int]
        L.mw_init.restype = None
        L.mw_init.argtypes = [C.c_int, C.c_int, C.c_int, _FP, _FP]
        L.mw_run_tile.restype = None
        L.mw_run_tile.argtypes = [C.c_int, C.c_long, C.c_int, C.c_int, C.c_float, _FP, _FP, _FP, _FP, _FP]
        L.mw_run_kernel.restype = None
        L.mw_run_kernel.argtypes = [C.c_int, C.c_long, C.c_long, C.c_int, C.c_int, C.c_float, _FP, _FP, _FP, _FP]
        L.mw_timestep.restype = None
        L.mw_timestep.argtypes = [C.c_int, C.c_int, C.c_float, _FP, _FP, _FP, _FP, C.c_int]
        L.mw_reductions.restype = None
        L.mw_reductions.argtypes = [C.c_int, C.c_int, _FP, _FP, C.POINTER(C.c_double), C.POINTER(C.c_double)]
        _ready = True
    return L


def _fp(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(_FP)


def kernel_ids(kernel, nx, nz):
    return _lib().mw_kernel_ids(kernel, nx, nz)


def kernel_tiles(kernel, nx, nz):
    return _lib().mw_kernel_tiles(kernel, nx, nz)


def kernel_of(kid):
    """kernel kind (HALO_X..UPDATE_Z) of kernel `kid` (0..35) of a time step"""
    step, sub = divmod(kid, 3)
    return (3 if step // 3 in (1, 2) else 0) + sub


class Sim:
    """State of one simulation: `state`, `state_tmp` (4, nz+4, nx+4), `flux` (4, nz+1, nx+1)."""

    def __init__(self, nx, nz, spec=COLLISION):
        L = _lib()
        self.nx, self.nz, self.spec = nx, nz, spec
        self.state = np.zeros((NUM_VARS, nz + 2 * HS, nx + 2 * HS), np.float32)
        self.hydro = np.zeros(L.mw_hydro_elems(nz), np.float32)
        L.mw_init(nx, nz, spec, _fp(self.state), _fp(self.hydro))
        self.state_tmp = self.state.copy()
        self.flux = np.zeros((NUM_VARS, nz + 1, nx + 1), np.float32)
        self.dt = L.mw_dt(nx, nz)
        self.dx, self.dz = L.mw_dx(nx), L.mw_dz(nz)

    def copy(self):
        s = object.__new__(Sim)
        s.__dict__.update(self.__dict__)
        s.state, s.state_tmp, s.flux, s.hydro = self.state.copy(), self.state_tmp.copy(), self.flux.copy(), self.hydro.copy()
        return s

    def timestep(self, start_from=0):
        _lib().mw_timestep(self.nx, self.nz, self.dt, _fp(self.state), _fp(self.state_tmp), _fp(self.flux), _fp(self.hydro), start_from)

    def run_kernel(self, kid, tile_lo=0, tile_hi=-1):
        _lib().mw_run_kernel(kid, tile_lo, tile_hi, self.nx, self.nz, self.dt, _fp(self.state), _fp(self.state_tmp), _fp(self.flux), _fp(self.hydro))

    def reductions(self):
        m, t = C.c_double(), C.c_double()
        _lib().mw_reductions(self.nx, self.nz, _fp(self.state), _fp(self.hydro), C.byref(m), C.byref(t))
        return m.value, t.value

    # views of the hydrostatic buffer
    def hy(self, name):
        nz = self.nz
        sizes = [("dens_cell", nz + 4), ("dens_theta_cell", nz + 4), ("dens_int", nz + 1), ("dens_theta_int", nz + 1), ("pressure_int", nz + 1), ("cell_const", 4)]
        off = 0
        for n, sz in sizes:
            if n == name:
                return self.hydro[off:off + sz]
            off += sz
        raise KeyError(name)
