"""Contraction tables of the linear Moment Tensor Potential, by level.

Host-side counterpart of the reference's ``MtpParam`` / ``mtpParamOp``
(source/descriptor/mtpr/src/mtpParam.cc:65-214, 435-469, 549-556;
src/mtpParamOp.cc:25-63): the tables are data, read either from an ``NN.almtp`` template
file (same search rule as the reference: ``$AI2POT_PATH/source/descriptor/mtpr/MTP_templates/``
or ``<package path>/_data/MTP_templates/``) or, when no template directory is available,
from the compact table archive packaged with this module (``_data/mtp_tables.npz``, levels
6-22, produced from the same MLIP-3 template files by ``tests/golden/make_mtp_tables.py``).
"""
import os
import re

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ai2pot_path = None
_cache = {}


class MtpError(RuntimeError):
    pass


def set_ai2pot_path(path):
    """Mirror of torch.ops.mtpr.set_ai2pot_path (source/descriptor/mtpr/bind/mtpr_bind.cc:31-36)."""
    global _ai2pot_path
    _ai2pot_path = path
    _cache.clear()


def template_dir():
    env = os.environ.get("AI2POT_PATH")
    if env:
        return os.path.join(env, "source", "descriptor", "mtpr", "MTP_templates")
    if _ai2pot_path:
        return os.path.join(_ai2pot_path, "_data", "MTP_templates")
    return None


def template_name(level):
    if level < 2 or level > 28 or level % 2 != 0:
        raise MtpError("mtp level must be an even number in 2..28")
    if level <= 4:
        return "depreciated-0%d.almtp" % level
    return "%02d.almtp" % level


def parse_almtp(path):
    """Parse one template file.  Like the reference, the first ten lines (species count,
    radial-basis header) are skipped: those values come from the model constructor."""
    try:
        with open(path) as fh:
            lines = fh.read().split("\n")
    except OSError:
        raise MtpError("Cannot open file " + path)
    body = "\n".join(lines[10:])

    def scalar(key):
        m = re.search(r"^\s*%s\s*=\s*(-?\d+)" % key, body, re.M)
        if not m:
            raise MtpError("Cannot read %s." % key)
        return int(m.group(1))

    def array(key, count, width):
        m = re.search(r"^\s*%s\s*=\s*(.*)$" % key, body, re.M)
        if not m:
            raise MtpError("Cannot read %s." % key)
        vals = np.array([int(x) for x in re.findall(r"-?\d+", m.group(1))], np.int32)
        if vals.size != count * width:
            raise MtpError("Cannot read %s." % key)
        return vals.reshape(count, width) if width > 1 else vals

    n_moms = scalar("alpha_moments_count")
    n_basic = scalar("alpha_index_basic_count")
    basic = array("alpha_index_basic", n_basic, 4)
    n_times = scalar("alpha_index_times_count")
    times = array("alpha_index_times", n_times, 4) if n_times else np.zeros((0, 4), np.int32)
    n_scalar = scalar("alpha_scalar_moments")
    mapping = array("alpha_moment_mapping", n_scalar, 1)
    return _finish(n_moms, basic, times, mapping)


def _finish(n_moms, basic, times, mapping):
    basic = np.ascontiguousarray(basic, np.int32).reshape(-1, 4)
    times = np.ascontiguousarray(times, np.int32).reshape(-1, 4)
    mapping = np.ascontiguousarray(mapping, np.int32)
    # set of radial-function indices each moment depends on (mtpParam.cc:435-469)
    mus = []
    by_dst = {}
    for m0, m1, _, dst in times:
        by_dst.setdefault(int(dst), []).append((int(m0), int(m1)))
    for i in range(n_moms):
        if i < basic.shape[0]:
            mus.append({int(basic[i, 0])})
        else:
            s = set()
            for m0, m1 in by_dst.get(i, ()):
                s |= mus[m0] | mus[m1]
            mus.append(s)
    width = max((len(s) for s in mus), default=0)
    mus4moms = -np.ones((n_moms, width), np.int32)
    for i, s in enumerate(mus):
        mus4moms[i, :len(s)] = sorted(s)
    return dict(alpha_moments_count=int(n_moms), alpha_index_basic=basic, alpha_index_times=times,
                alpha_moment_mapping=mapping,
                num_mus4moms=np.array([len(s) for s in mus], np.int32), mus4moms=mus4moms,
                nmus=int(basic[:, 0].max()) + 1 if basic.size else 1)


def mtp_param(level):
    """Tables of one MTP level as a dict of int32 NumPy arrays (the seven outputs of the
    reference's ``mtpParamOp`` plus nothing else)."""
    level = int(level)
    if level in _cache:
        return _cache[level]
    name = template_name(level)
    d = template_dir()
    if d is not None and os.path.exists(os.path.join(d, name)):
        out = parse_almtp(os.path.join(d, name))
    else:
        arch = os.path.join(_HERE, "_data", "mtp_tables.npz")
        with np.load(arch) as z:
            key = "L%02d" % level
            if key + "_basic" not in z:
                raise MtpError("Cannot open file %s (and level %d is not in the packaged tables)"
                               % (name, level))
            out = _finish(int(z[key + "_count"]), z[key + "_basic"], z[key + "_times"],
                          z[key + "_mapping"])
    _cache[level] = out
    return out


def write_almtp(path, t):
    """Write tables in the template text format (ten header lines, then the six table
    entries), e.g. to materialise a template directory from the packaged archive."""
    def rows(a):
        return "{" + ", ".join("{" + ", ".join(str(int(v)) for v in r) + "}" for r in a) + "}"
    header = ["MTP", "version = 1.1.0", "potential_name = MTP1m", "species_count = 1", "potential_tag = ",
              "radial_basis_type = RBChebyshev", "\tmin_dist = 2", "\tmax_dist = 5", "\tradial_basis_size = 8",
              "\tradial_funcs_count = %d" % t["nmus"]]
    body = ["alpha_moments_count = %d" % t["alpha_moments_count"],
            "alpha_index_basic_count = %d" % t["alpha_index_basic"].shape[0],
            "alpha_index_basic = " + rows(t["alpha_index_basic"]),
            "alpha_index_times_count = %d" % t["alpha_index_times"].shape[0],
            "alpha_index_times = " + rows(t["alpha_index_times"]),
            "alpha_scalar_moments = %d" % t["alpha_moment_mapping"].size,
            "alpha_moment_mapping = {" + ", ".join(str(int(v)) for v in t["alpha_moment_mapping"]) + "}"]
    with open(path, "w") as fh:
        fh.write("\n".join(header + body) + "\n")


def validate_tables(t):
    """Host-side checks the kernels rely on; raises MtpError on violation."""
    n = t["alpha_moments_count"]
    basic, times, mapping = t["alpha_index_basic"], t["alpha_index_times"], t["alpha_moment_mapping"]
    nb = basic.shape[0]
    if nb > n or (basic < 0).any():
        raise MtpError("alpha_index_basic out of range")
    if times.size:
        if (times[:, [0, 1, 3]] < 0).any() or (times[:, [0, 1, 3]] >= n).any():
            raise MtpError("alpha_index_times refers to a moment outside [0, alpha_moments_count)")
        if (times[:, 3] < nb).any():
            raise MtpError("alpha_index_times writes into a basic moment")
    if mapping.size and ((mapping < 0).any() or (mapping >= n).any()):
        raise MtpError("alpha_moment_mapping out of range")
