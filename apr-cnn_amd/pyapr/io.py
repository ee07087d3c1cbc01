"""File I/O for APRs and particle fields: ``read`` / ``write`` / ``read_particles`` / ``write_particles`` /
``get_particle_names`` with the call signatures of pyapr/io/io_api.py:20-400 (time point and channel arguments
are accepted and must stay at their defaults).

The reference stores HDF5 through LibAPR's APRFile, which is not part of the reference tree; the container here
is a NumPy ``.npz`` archive (read with ``allow_pickle=False``) that holds the state of BindAPR.hpp:72-90 -
``org_dims``, ``xz_end_vec`` / ``y_vec`` of particles and tree - plus one array ``parts/<name>`` per particle field
and ``tree_parts/<name>`` per tree field.  The file name is used as given (``.apr`` included): NumPy's own suffix
rule is bypassed by writing through an open file object."""
import os
import zipfile
import numpy as np

from .data_containers import APR, APRParameters

__all__ = ["read", "read_apr", "read_particles", "write", "write_apr", "write_particles", "get_particle_names",
           "get_particle_type"]

_PARAM_FIELDS = ("rel_error", "gradient_smoothing", "Ip_th", "sigma_th", "grad_th", "dz", "dx", "dy")


def _check_defaults(t, channel_name):
    if t != 0 or channel_name != "t":
        raise ValueError("this container holds one time point and one channel (t=0, channel_name='t')")


def _load(fpath):
    if not os.path.isfile(fpath):
        raise ValueError(f"Invalid path {fpath} - file does not exist")
    return np.load(fpath, allow_pickle=False)


def _save(fpath, arrays):
    with open(fpath, "wb") as f:
        np.savez(f, **arrays)


def _apr_arrays(apr):
    oy, ox, oz, par, xze, yv, txze, tyv = apr.get_state()
    return {"org_dims": np.array([oy, ox, oz], np.int64), "xz_end_vec": xze, "y_vec": yv,
            "tree_xz_end_vec": txze, "tree_y_vec": tyv,
            "parameters": np.array([float(getattr(par, k)) for k in _PARAM_FIELDS], np.float64),
            "name": np.array(apr.name)}


def _apr_from(z):
    par = APRParameters()
    for k, v in zip(_PARAM_FIELDS, z["parameters"]):
        setattr(par, k, float(v))
    apr = APR.from_state(z["org_dims"], z["xz_end_vec"], z["y_vec"], z["tree_xz_end_vec"], z["tree_y_vec"], par)
    apr.name = str(z["name"])
    return apr


def write(fpath, apr, parts, t=0, channel_name="t", parts_name="particles", write_linear=True, write_tree=True,
          tree_parts=None):
    """io_api.py:73-131.  The tree access is always stored (the operators need it), whatever ``write_tree`` says."""
    if not fpath:
        print("Empty path given. Ignoring call to pyapr.io.write")
        return
    _check_defaults(t, channel_name)
    parts = np.asarray(parts)
    if parts.shape != (apr.total_number_particles(),):
        raise ValueError(f"particle field of size {parts.shape} does not match the APR ({apr.total_number_particles()})")
    arrays = _apr_arrays(apr)
    arrays["parts/" + parts_name] = parts
    if tree_parts is not None:
        arrays["tree_parts/" + parts_name] = np.asarray(tree_parts)
    _save(fpath, arrays)


def write_apr(fpath, apr, t=0, channel_name="t", write_linear=True, write_tree=True):
    """io_api.py:238-285."""
    if not fpath:
        print("Empty path given. Ignoring call to pyapr.io.write_apr")
        return
    _check_defaults(t, channel_name)
    _save(fpath, _apr_arrays(apr))


def write_particles(fpath, parts, t=0, channel_name="t", parts_name="particles", tree=False, append=True):
    """io_api.py:134-178: adds (append=True) a field to an existing file, or starts a new file holding only it."""
    if not fpath:
        print("Empty path given. Ignoring call to pyapr.io.write_particles")
        return
    _check_defaults(t, channel_name)
    arrays = {}
    if append and os.path.isfile(fpath):
        with _load(fpath) as z:
            arrays = {k: z[k] for k in z.files}
    arrays[("tree_parts/" if tree else "parts/") + parts_name] = np.asarray(parts)
    _save(fpath, arrays)


def read(fpath, apr=None, parts=None, t=0, channel_name="t", parts_name="particles"):
    """io_api.py:20-70.  Returns ``(apr, parts)``; ``parts`` is a NumPy array of the stored type."""
    _check_defaults(t, channel_name)
    with _load(fpath) as z:
        if "parts/" + parts_name not in z.files:
            raise ValueError(f"no particle field '{parts_name}' in {fpath}")
        new = _apr_from(z)
        data = z["parts/" + parts_name]
    if apr is not None:
        apr.__dict__.update(new.__dict__); new._plans = {}
        new = apr
    if parts is not None:
        if parts.dtype != data.dtype:
            raise ValueError(f"particle type mismatch: file holds {data.dtype}, {parts.dtype} was given")
        parts.resize(data.shape, refcheck=False); parts[...] = data
        data = parts
    return new, data


def read_apr(fpath, apr=None, t=0, channel_name="t"):
    """io_api.py:288-323."""
    _check_defaults(t, channel_name)
    with _load(fpath) as z:
        new = _apr_from(z)
    if apr is not None:
        apr.__dict__.update(new.__dict__); new._plans = {}
        new = apr
    return new


def read_particles(fpath, parts=None, t=0, channel_name="t", parts_name="particles", tree=False):
    """io_api.py:181-235."""
    _check_defaults(t, channel_name)
    key = ("tree_parts/" if tree else "parts/") + parts_name
    with _load(fpath) as z:
        if key not in z.files:
            raise ValueError(f"no particle field '{parts_name}' in {fpath}")
        data = z[key]
    if parts is not None:
        if parts.dtype != data.dtype:
            raise ValueError(f"particle type mismatch: file holds {data.dtype}, {parts.dtype} was given")
        parts.resize(data.shape, refcheck=False); parts[...] = data
        data = parts
    return data


def get_particle_names(fpath, t=0, channel_name="t", tree=False):
    """Names of the stored particle fields (io_api.py:326-360)."""
    _check_defaults(t, channel_name)
    prefix = "tree_parts/" if tree else "parts/"
    with zipfile.ZipFile(fpath) as z:
        names = [n[:-4] for n in z.namelist() if n.endswith(".npy")]
    return [n[len(prefix):] for n in names if n.startswith(prefix)]


def get_particle_type(fpath, t=0, channel_name="t", parts_name="particles", tree=False):
    """Stored type of a field as the reference names them (io_api.py:363-400)."""
    data = read_particles(fpath, t=t, channel_name=channel_name, parts_name=parts_name, tree=tree)
    names = {np.dtype(np.uint8): "uint8", np.dtype(np.uint16): "uint16", np.dtype(np.uint64): "uint64",
             np.dtype(np.float32): "float"}
    return names.get(data.dtype, str(data.dtype))
