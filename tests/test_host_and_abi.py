"""CPU-only checks: the synthetic generators are deterministic, the MTP tables parse and match
the template sizes, argument validation of the host-side operator mirror fires before any
GPU work, and libai2pot_hip.so loads and exports every symbol include/ai2pot_hip.h declares
(no compute call is made here)."""
import ctypes
import os
import re

import numpy as np
import pytest

from ai2pot_amd import mtp_param, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_rng_is_deterministic_and_sane():
    a = synth.rng_uniform(5, 1000)
    assert np.array_equal(a, synth.rng_uniform(5, 1000))
    assert np.array_equal(a[10:20], synth.rng_uniform(5, 10, offset=10))
    assert not np.array_equal(a, synth.rng_uniform(6, 1000))
    assert 0.45 < a.mean() < 0.55 and a.min() >= 0 and a.max() < 1
    n = synth.rng_normal(7, 20000)
    assert abs(n.mean()) < 0.03 and abs(n.std() - 1) < 0.03
    # frozen values: the generator must not drift between NumPy versions
    assert synth.rng_bits(1, 2).tolist() == [3243820990799439115, 18353093357008240898]
    assert synth.rng_uniform(1001, 1)[0] == 0.08327232503302318
    assert abs(synth.rng_normal(7, 1)[0] - 0.5744747071993579) < 1e-15


def test_structures():
    lat, pos = synth.diamond_cell()
    assert pos.shape == (216, 3) and abs(lat[0, 0] - 16.29) < 1e-12
    lat, pos = synth.fcc_cell(4, 4.949, 0.15, 3)
    assert pos.shape == (256, 3) and (pos >= 0).all() and (pos < lat[0, 0]).all()
    lat, pos = synth.random_packed(100, [12.0, 12.0, 12.0], 2.2, 9)
    d = pos[:, None, :] - pos[None, :, :]
    d -= 12.0 * np.round(d / 12.0)
    r = np.sqrt((d * d).sum(-1)) + 10 * np.eye(100)
    assert r.min() >= 2.2


@pytest.mark.parametrize("level,sizes", [(10, (41, 25, 42, 16, 3)), (16, (350, 130, 969, 92, 4)),
                                         (20, (1352, 295, 6349, 288, 5))])
def test_mtp_tables(level, sizes, monkeypatch):
    """Counts of the MLIP-3 templates (e.g. MTP_templates/10.almtp:10-16) and nmus = 1 + max mu
    (mtpr/tests/test_mtpParam.cc:140 asserts nmus == 5 for level 20)."""
    monkeypatch.delenv("AI2POT_PATH", raising=False)
    mtp_param.set_ai2pot_path(None)
    t = mtp_param.mtp_param(level)
    assert (t["alpha_moments_count"], t["alpha_index_basic"].shape[0], t["alpha_index_times"].shape[0],
            t["alpha_moment_mapping"].size, t["nmus"]) == sizes
    mtp_param.validate_tables(t)
    assert t["num_mus4moms"].shape == (sizes[0],) and t["mus4moms"].shape[0] == sizes[0]
    assert (t["alpha_index_times"][:, 3] >= sizes[1]).all()
    with pytest.raises(mtp_param.MtpError):
        mtp_param.mtp_param(7)
    with pytest.raises(mtp_param.MtpError):
        mtp_param.mtp_param(26)          # not packaged and no template directory configured


def test_mtp_template_parser(tmp_path, monkeypatch):
    """The .almtp reader skips ten header lines, like the reference (mtpParam.cc:92-93)."""
    text = "\n".join(["h"] * 10 + [
        "alpha_moments_count = 4", "alpha_index_basic_count = 2",
        "alpha_index_basic = {{0, 0, 0, 0}, {1, 1, 0, 0}}", "alpha_index_times_count = 2",
        "alpha_index_times = {{0, 0, 1, 2}, {1, 1, 3, 3}}", "alpha_scalar_moments = 3",
        "alpha_moment_mapping = {0, 2, 3}", ""])
    d = tmp_path / "source" / "descriptor" / "mtpr" / "MTP_templates"
    d.mkdir(parents=True)
    (d / "06.almtp").write_text(text)
    monkeypatch.setenv("AI2POT_PATH", str(tmp_path))
    mtp_param.set_ai2pot_path(None)
    t = mtp_param.mtp_param(6)
    assert t["alpha_moments_count"] == 4 and t["nmus"] == 2
    assert t["alpha_index_times"].tolist() == [[0, 0, 1, 2], [1, 1, 3, 3]]
    assert t["mus4moms"].tolist() == [[0], [1], [0], [1]]
    (d / "08.almtp").write_text("broken")
    with pytest.raises(mtp_param.MtpError):
        mtp_param.mtp_param(8)
    monkeypatch.delenv("AI2POT_PATH")
    mtp_param.set_ai2pot_path(None)


def test_operator_mirror_rejects_host_tensors():
    import torch
    from ai2pot_amd import nblist, ops
    z = torch.zeros
    with pytest.raises(RuntimeError):        # no CPU path: the product never falls back
        ops.nepToEFVOp(8, 6, 4, 4, z(720), z(3300), z(150), z(150), z(3), z(1, dtype=torch.int32),
                       z(1, 4, dtype=torch.int32), z(1, 4, dtype=torch.int32), z(1, 4, 10, dtype=torch.int32),
                       z(1, 4, 10, 3), z(1, 4, dtype=torch.int32), z(3, dtype=torch.int32), 0, 7.0, 4.0,
                       z(22), 0.0, 0.0, None, None)
    lat, types, frac = synth.mos2_fixture()
    with pytest.raises(TypeError):
        nblist.find_info4mlff(lat, types, frac, 5, 20, False, [True, True, True], False)
    with pytest.raises(TypeError):
        nblist.find_info4mlff(lat, types, frac, 5.0, 20.0, False, [True, True, True], False)


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ai2pot_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(a2p_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    path = os.path.join(ROOT, "ai2pot_amd", "libai2pot_hip.so")
    if not os.path.exists(path):
        pytest.fail("ai2pot_amd/libai2pot_hip.so is missing: run `python -m ai2pot_amd.build`")
    names = declared_symbols()
    assert "a2p_nep_efv_f32" in names and "a2p_nblist_build_f32" in names
    try:
        lib = ctypes.CDLL(path)
    except OSError as ex:
        pytest.skip("the HIP runtime cannot be loaded in this environment: %s" % ex)
    for n in names:
        assert hasattr(lib, n), "%s is declared in include/ai2pot_hip.h but not exported" % n
    lib.a2p_abi_version.restype = ctypes.c_int
    assert lib.a2p_abi_version() >= 1


def test_staged_rows_never_load_past_the_arrays():
    """Index arithmetic of the staging kernel's row loads (csrc/nep_staged.hip: staged_row_index and
    the slot choice of staged_load), emulated on the host: whatever natoms_pad is, every address the
    256 threads of the last workgroup form lies inside the caller's [B, P, U] arrays."""
    SB, SCH = 256, 8
    for B, P, U in ((1, 1, 8), (1, 96, 200), (2, 257, 16), (3, 42592 % 1024 + 3, 200), (2, 512, 8)):
        for b in range(B):
            for blk in range((P + SB - 1) // SB):
                rowbase = b * P + blk * SB
                for tid in range(0, SB, 7):
                    for it in range(SCH):
                        e = it * SB + tid
                        la, slot = e // SCH, e % SCH + 192
                        have = blk * SB + la < P and slot < U          # rows past P hold no neighbours
                        row = min(rowbase + la, b * P + P - 1)
                        pr = row * U + (slot if have else 0)
                        assert 0 <= pr < B * P * U
                        assert row // P == b                            # never another structure's row


# Positional argument types of the operators the reference registers (i = int, f = float, T = Tensor, s = str), read
# off its TORCH_LIBRARY blocks; the number is the line of the m.def in
# source/descriptor/{nep,mtpr,nnmtp}/bind/*_bind.cc and source/fvt/bind/fvt_sr_op_bind.cc.
REFERENCE_SCHEMAS = {
    ("nep", "nepToEFOp"): ("iiiiTTTTTTTTTTTTiffTffTT", 25),
    ("nep", "nepToEFVOp"): ("iiiiTTTTTTTTTTTTiffTffTT", 80),
    ("nep", "nepToEFLossOp"): ("ffTTiiiiTTTTTTTTTTTTiffTffTT", 135),
    ("nep", "nepToLossOp"): ("fffTTTiiiiTTTTTTTTTTTTiffTffTT", 204),
    ("nep", "nepToDescriptorsOp"): ("iiiiTTTTTTTTiff", 277),
    ("mtpr", "set_ai2pot_path"): ("s", 31),
    ("mtpr", "CoeffsSchmidtOrthOp"): ("iiiT", 38),
    ("mtpr", "LinMatrixLinVectorOp"): ("fffTTTifTTTiTTTiTTTTTTTiffTffTT", 57),
    ("mtpr", "mtpParamOp"): ("i", 131),
    ("mtpr", "mtpBasisOp"): ("TTTTTTiifTTTTTTTiff", 140),
    ("mtpr", "linearMtpToLossOp"): ("fffTTTifTTTiTTTiTTTTTTTiffTffTT", 189),
    ("mtpr", "linearMtpToEFLossOp"): ("ffTTifTTTiTTTiTTTTTTTiffTffTT", 263),
    ("mtpr", "linearMtpToEFVOp"): ("ifTTTiTTTiTTTTTTTiffTffTT", 333),
    ("mtpr", "linearMtpToEFOp"): ("ifTTTiTTTiTTTTTTTiffTffTT", 396),
    ("mtpr", "linearMtpToEsitesOp"): ("ifTTTiTTTiTTTTTTTiffTffTT", 459),
    ("mtpr", "linearMtpToDescriptorsOp"): ("ifTiTTTiTTTTTTTiff", 521),
    ("nnmtp", "set_ai2pot_path"): ("s", 27),
    ("nnmtp", "mtpParamOp"): ("i", 34),
    ("nnmtp", "nnMtpToEFLossOp"): ("ffTTiTTTTiTTTiTTTTTTTiffTTffTT", 43),
    ("nnmtp", "nnMtpToLossOp"): ("fffTTTiTTTTiTTTiTTTTTTTiffTTffTT", 116),
    ("nnmtp", "nnMtpToEFOp"): ("iTTTTiTTTiTTTTTTTiffTTffTT", 193),
    ("nnmtp", "nnMtpToEFVOp"): ("iTTTTiTTTiTTTTTTTiffTTffTT", 258),
    ("nnmtp", "nnMtpToDescriptorsOp"): ("iTiTTTiTTTTTTTiff", 323),
    ("nnmtp", "nnMtpToEsitesOp"): ("iTTTTiTTTiTTTTTTTiffTTffTT", 370),
    ("fvt", "ForceSrOp"): ("TTTTiiT", 10),
    ("fvt", "VirialSrOp"): ("TTiT", 32),
}


def test_bind_libraries_register_the_reference_operators():
    """The operator libraries load without a GPU and register every operator of the reference under its name with
    its positional argument types (what TorchScript-exported models and ai2pot/fromcc bind to)."""
    import glob
    import torch
    import ai2pot_amd
    libdir = os.path.join(os.path.dirname(os.path.abspath(ai2pot_amd.__file__)), "_lib")
    libs = sorted(glob.glob(os.path.join(libdir, "lib*_bind.so")))
    assert {os.path.basename(p) for p in libs} >= {"libnep_bind.so", "libmtpr_bind.so", "libnnmtp_bind.so",
                                                   "libfvt_sr_op_bind.so", "libnblist_bind.so"}
    for p in libs:
        torch.ops.load_library(p)
    code = {"int": "i", "float": "f", "Tensor": "T", "str": "s", "Optional[Tensor]": "T"}
    for (ns, name), (want, _) in REFERENCE_SCHEMAS.items():
        op = getattr(getattr(torch.ops, ns), name)
        schema = op.default._schema
        got = "".join(code.get(str(a.type), "?") for a in schema.arguments)
        assert got == want, (ns, name, got, want)


def test_nblist_module_checks_its_arguments_like_the_reference():
    """The CPython module `nblist` (source/nblist/bind/nblist_bind.cc:46-69): eight positional arguments, a
    TypeError for an argument of the wrong kind, raised before any device work."""
    import importlib
    import sys
    import ai2pot_amd
    libdir = os.path.join(os.path.dirname(os.path.abspath(ai2pot_amd.__file__)), "_lib")
    sys.path.insert(0, libdir)
    try:
        mod = importlib.import_module("nblist")
    finally:
        sys.path.remove(libdir)
    assert hasattr(mod, "find_info4mlff")
    lat = np.eye(3) * 10.0
    ty = np.zeros(2, np.int32)
    pos = np.zeros((2, 3))
    good = [lat, ty, pos, 5.0, 20, True, [True, True, True], False]
    for i, bad in [(0, [1.0]), (1, [0, 0]), (2, "x"), (3, 5), (4, 20.0), (5, 1), (6, (True, True, True)), (7, 0)]:
        args = list(good)
        args[i] = bad
        with pytest.raises(TypeError):
            mod.find_info4mlff(*args)
    with pytest.raises(TypeError):
        mod.find_info4mlff(*good[:7])
