"""APR container: the linear-access arrays of the particles and of the APR tree.

Mirrors the members of the reference's ``APR`` / ``LinearIterator`` bindings that the network
operators and models call (pyapr/data_containers/src/BindAPR.hpp:46-63,
BindLinearIterator.hpp:70-92).  The serialisable state is the one of BindAPR.hpp:72-90:
``org_dims``, ``xz_end_vec`` (uint64) and ``y_vec`` (uint16) for particles and tree;
``level_xz_vec`` is recomputed from the dimensions.
"""
import ctypes as C
import numpy as np

from . import _native


class APRParameters:
    """Subset of pyapr/data_containers/src/BindParameters.hpp:18-29 used by the builder."""

    def __init__(self):
        self.rel_error = 0.1
        self.gradient_smoothing = 3.0
        self.Ip_th = 0.0
        self.sigma_th = 0.0
        self.grad_th = 0.0
        self.auto_parameters = False
        self.dz = self.dx = self.dy = 1.0
        self.name = ""


class LinearIterator:
    """Read-only view of one access (particles or tree)."""

    def __init__(self, level_min, level_max, z_num, x_num, y_num, level_xz_vec, xz_end_vec, y_vec, lmax_all):
        self._lmin, self._lmax = int(level_min), int(level_max)
        self._z, self._x, self._y = z_num, x_num, y_num
        self.level_xz_vec, self.xz_end_vec, self.y_vec = level_xz_vec, xz_end_vec, y_vec
        self._lmax_all = lmax_all
        self._row_end = 0

    def level_min(self): return self._lmin
    def level_max(self): return self._lmax
    def x_num(self, level): return int(self._x[level])
    def y_num(self, level): return int(self._y[level])
    def z_num(self, level): return int(self._z[level])
    def level_size(self, level): return 1 << (self._lmax_all - level)

    def particles_level_begin(self, level):
        level = min(max(level, 0), self._lmax + 1)
        return int(self.xz_end_vec[int(self.level_xz_vec[level]) - 1])

    def particles_level_end(self, level):
        if level < self._lmin:
            return 0
        level = min(level, self._lmax)
        return int(self.xz_end_vec[int(self.level_xz_vec[level + 1]) - 1])

    def total_number_particles(self, level=0):
        """Number of particles up to and including ``level`` (0 -> all levels)."""
        if level == 0:
            return int(self.y_vec.shape[0])
        return self.particles_level_end(level)

    def begin(self, level, z, x):
        row = int(self.level_xz_vec[level]) + x + z * self.x_num(level)
        self._row_end = int(self.xz_end_vec[row])
        return int(self.xz_end_vec[row - 1])

    def end(self): return self._row_end
    def y(self, idx): return int(self.y_vec[idx])


def _level_tables(org_z, org_x, org_y, level_min, level_max, lmax_all):
    z = np.ones(lmax_all + 1, np.int32); x = z.copy(); y = z.copy()
    for l in range(lmax_all + 1):
        s = lmax_all - l
        z[l] = (org_z + (1 << s) - 1) >> s
        x[l] = (org_x + (1 << s) - 1) >> s
        y[l] = (org_y + (1 << s) - 1) >> s
    lxz = np.ones(level_max + 2, np.uint64)
    counter = 1
    for l in range(level_max + 1):
        lxz[l] = counter
        if l >= level_min:
            counter += int(x[l]) * int(z[l])
    lxz[level_max + 1] = counter
    return z, x, y, lxz


class APR:
    """An APR as the operators see it.  Build with :func:`pyapr.converter.get_apr`,
    :meth:`from_level_field` or :meth:`from_state`."""

    def __init__(self):
        self.name = ""
        self._org = (1, 1, 1)          # (z, x, y)
        self._lmax = 1
        self._acc = None               # LinearIterator for particles
        self._tree = None              # LinearIterator for the tree
        self._params = APRParameters()
        self._plans = {}               # device index -> native plan handle
        self._keep = None

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_level_field(cls, shape, desired):
        """Build from a required-level field given on the level (level_max-1) grid.

        ``shape`` = (z, x, y) of the image; ``desired`` uint8 array with the dims of
        :meth:`level_dims` ``(level_max-1)``; cell value v asks for particles of level >= v
        somewhere inside the cell (0 = no requirement).  Used by the converter and by tests
        (random fields give random valid APRs).
        """
        lib = _native.core()
        z, x, y = (int(v) for v in shape)
        h = lib.aprcore_create(z, x, y)
        if not h:
            raise ValueError(lib.aprcore_last_error().decode())
        try:
            lmax = lib.aprcore_level_max(h)
            dims = np.zeros(3, np.int32)
            lib.aprcore_level_dims(h, lmax - 1, dims.ctypes.data)
            desired = np.ascontiguousarray(desired, dtype=np.uint8)
            if desired.size != int(dims.prod()):
                raise ValueError(f"desired level field must have {tuple(dims)} cells, got {desired.shape}")
            lib.aprcore_build_from_levels(h, desired.ctypes.data)
            return cls._from_handle(h, (z, x, y))
        finally:
            lib.aprcore_destroy(h)

    @classmethod
    def _from_handle(cls, h, shape):
        lib = _native.core()
        self = cls()
        self._org = tuple(shape)
        self._lmax = lib.aprcore_level_max(h)
        its = []
        for which in (0, 1):
            info = np.zeros(4, np.int64)
            lib.aprcore_access_info(h, which, info.ctypes.data)
            lmin, lmax, nrows, n = (int(v) for v in info)
            zn = np.zeros(self._lmax + 1, np.int32); xn = zn.copy(); yn = zn.copy()
            lxz = np.zeros(lmax + 2, np.uint64)
            xze = np.zeros(nrows, np.uint64)
            yv = np.zeros(max(n, 1), np.uint16)[:n]
            lib.aprcore_access_copy(h, which, zn.ctypes.data, xn.ctypes.data, yn.ctypes.data,
                                    lxz.ctypes.data, xze.ctypes.data, yv.ctypes.data if n else None)
            its.append(LinearIterator(lmin, lmax, zn, xn, yn, lxz, xze, yv, self._lmax))
        self._acc, self._tree = its
        return self

    @classmethod
    def from_state(cls, org_dims_yxz, xz_end_vec, y_vec, tree_xz_end_vec, tree_y_vec, parameters=None):
        """Rebuild from the pickled state of the reference's APR (BindAPR.hpp:72-131):
        ``(org_dims(0)=y, org_dims(1)=x, org_dims(2)=z)``, ``xz_end_vec``/``y_vec`` of the
        particles and of the tree."""
        oy, ox, oz = (int(v) for v in org_dims_yxz)
        self = cls()
        self._org = (oz, ox, oy)
        m, lmax = max(oz, ox, oy), 0
        while (1 << lmax) < m:
            lmax += 1
        self._lmax = max(lmax, 1)
        for name, lmin, lm, xze, yv in (("_acc", 1, self._lmax, xz_end_vec, y_vec),
                                        ("_tree", 0, self._lmax - 1, tree_xz_end_vec, tree_y_vec)):
            zn, xn, yn, lxz = _level_tables(oz, ox, oy, lmin, lm, self._lmax)
            xze = np.ascontiguousarray(xze, np.uint64); yv = np.ascontiguousarray(yv, np.uint16)
            if xze.shape[0] != int(lxz[-1]):
                raise ValueError("xz_end_vec does not match the row table implied by the dimensions")
            setattr(self, name, LinearIterator(lmin, lm, zn, xn, yn, lxz, xze, yv, self._lmax))
        if parameters is not None:
            self._params = parameters
        return self

    def get_state(self):
        return (self._org[2], self._org[1], self._org[0], self._params, self._acc.xz_end_vec, self._acc.y_vec,
                self._tree.xz_end_vec, self._tree.y_vec)

    # pickle support with the reference's state tuple (BindAPR.hpp:67-131); device plans are rebuilt on demand
    def __getstate__(self):
        if self._acc is None:
            raise RuntimeError("Invalid state - APR not initialized")
        return self.get_state() + (self.name,)

    def __setstate__(self, t):
        if len(t) not in (8, 9):
            raise RuntimeError("Error unpickling APR object - invalid state size")
        other = APR.from_state(t[0:3], t[4], t[5], t[6], t[7], parameters=t[3])
        self.__dict__.update(other.__dict__)
        other._plans = {}
        self.name = t[8] if len(t) == 9 else ""

    def particle_levels(self):
        """Level of every particle, uint8 (what ParticleData.fill_with_levels writes, used by the collate function of
        apr_models/utils/dataset.py:147-151)."""
        out = np.empty(self.total_number_particles(), np.uint8)
        for level in range(self.level_min(), self.level_max() + 1):
            out[self._acc.particles_level_begin(level):self._acc.particles_level_end(level)] = level
        return out

    # ------------------------------------------------------------------ reference API
    def __repr__(self):
        return "APR(shape [{}, {}, {}], {} particles)".format(*self._org, self.total_number_particles())

    def total_number_particles(self): return self._acc.total_number_particles()
    def total_number_tree_particles(self): return self._tree.total_number_particles()
    def level_min(self): return self._acc.level_min()
    def level_max(self): return self._acc.level_max()
    def x_num(self, level): return self._acc.x_num(level)
    def y_num(self, level): return self._acc.y_num(level)
    def z_num(self, level): return self._acc.z_num(level)
    def iterator(self): return self._acc
    def tree_iterator(self): return self._tree
    def org_dims(self, dim): return (self._org[2], self._org[1], self._org[0])[dim]
    def shape(self): return self._org
    def get_parameters(self): return self._params

    def computational_ratio(self):
        return float(np.prod(self._org)) / max(self.total_number_particles(), 1)

    def level_dims(self, level):
        return (self._acc.z_num(level), self._acc.x_num(level), self._acc.y_num(level))

    # ------------------------------------------------------------------ device side
    def _desc(self, it):
        d = _native.AccessDesc()
        d.level_min, d.level_max = it.level_min(), it.level_max()
        d.z_num, d.x_num, d.y_num = it._z.ctypes.data, it._x.ctypes.data, it._y.ctypes.data
        d.level_xz_vec = it.level_xz_vec.ctypes.data
        d.xz_end_vec = it.xz_end_vec.ctypes.data
        d.y_vec = it.y_vec.ctypes.data if it.y_vec.shape[0] else None
        d.n_rows = it.xz_end_vec.shape[0]
        d.n_particles = it.y_vec.shape[0]
        return d

    def init_cuda(self, with_tree=True, device=None):
        """Upload the access structure and derived index tables to the GPU (cached per device).
        Name kept from the reference (BindAPR.hpp:63); on PyTorch-ROCm "cuda" is the HIP device."""
        import torch
        dev = torch.cuda.current_device() if device is None else torch.device(device).index or 0
        if dev not in self._plans:
            lib = _native.hip()
            h = C.c_void_p()
            a, t = self._desc(self._acc), self._desc(self._tree)
            rc = lib.aprnet_plan_create(C.byref(a), C.byref(t), dev, C.byref(h))
            if rc != 0:
                raise RuntimeError("aprnet_plan_create failed: " + lib.aprnet_last_error().decode())
            self._plans[dev] = h
        return self

    def plan(self, device_index):
        if device_index not in self._plans:
            self.init_cuda(device=f"cuda:{device_index}")
        return self._plans[device_index]

    def __del__(self):
        try:
            lib = _native.hip() if self._plans else None
            for h in self._plans.values():
                lib.aprnet_plan_destroy(h)
        except Exception:
            pass


class APRPtrVector(list):
    """The reference passes ``APRPtrVector(aprs)`` (a bound std::vector<APR*>, BindAPR.hpp:133)
    into native calls; a plain list plays that role here."""
