"""The C-ABI library builds, loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    hdr = open(os.path.join(ROOT, "include", "pccnn_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(pccnn_\w+)\s*\(([^;]*?)\)\s*;", hdr, flags=re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args == "void" else len(args.split(","))
    return out


@pytest.fixture(scope="module")
def lib_path():
    from pccnn_lib_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH):
        build.build(verbose=False)
    return _lib.LIB_PATH


def test_every_declared_symbol_is_exported(lib_path):
    lib = ctypes.CDLL(lib_path)
    declared = _declared()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), name


def test_ctypes_table_matches_header(lib_path):
    from pccnn_lib_amd import _lib
    declared = _declared()
    assert set(declared) == set(_lib.SIGNATURES)
    for name, nargs in declared.items():
        assert len(_lib.SIGNATURES[name][1]) == nargs, name


def test_argument_validation_needs_no_gpu(lib_path):
    # Host-side checks run before any kernel launch, so they can be exercised on a CPU-only machine.
    from pccnn_lib_amd import _lib
    lib = _lib.load()
    assert lib.pccnn_version() == 1
    for bad in (1, 7):
        rc = lib.pccnn_compute_keys(None, None, None, None, None, 10, bad, None, None)
        assert rc == -2 and b"d=%d" % bad in lib.pccnn_last_error()
    rc = lib.pccnn_compute_keys(None, None, None, None, None, 10, 2, None, None)
    assert rc == -1 and b"null" in lib.pccnn_last_error()
    rc = lib.pccnn_compute_keys(None, None, None, None, None, 10, 3, None, None)
    assert rc == -1 and b"null" in lib.pccnn_last_error()
    assert lib.pccnn_compute_keys(None, None, None, None, None, 0, 3, None, None) == 0
    rc = lib.pccnn_sort_keys(ctypes.c_void_p(16), 100, 20, ctypes.c_void_p(16), ctypes.c_void_p(16), None, 3, None,
                             None, 0, None)
    assert rc == -3 and b"workspace" in lib.pccnn_last_error()
    rc = lib.pccnn_kpconv_forward(None, None, None, None, None, None, None, 0.5, None, 10, 10, 10, 3, 8, 65, 8, None,
                                  None, None, 0, None)
    assert rc == -2 and b"k=65" in lib.pccnn_last_error()
    from pccnn_lib_amd import pccnn_lib_ops as ops
    desc = _lib.Basis()
    desc.kind = 9
    rc = lib.pccnn_conv_forward(ctypes.byref(desc), None, None, None, None, None, None, None, 10, 10, 10, 3, 8, 1, 8,
                                0, None, None, None, 0, None)
    assert rc == -1 and b"basis kind 9" in lib.pccnn_last_error()
    desc.kind, desc.nb0, desc.nb1, desc.nb2 = ops.BASIS_SPH, 4, 4, 4
    desc.a = desc.b = desc.c = 16
    rc = lib.pccnn_conv_weight_var(ctypes.byref(desc), None, None, None, None, None, None, 10, 10, 10, 3, 8, 0, None,
                                   None, 0, None)
    assert rc == -2 and b"k=65" in lib.pccnn_last_error()
    rc = lib.pccnn_grid_build(None, None, None, None, None, 10, 9, 20, 4, 0, None, None, None, None, None, None, None,
                              0, None)
    assert rc == -2 and b"d=9" in lib.pccnn_last_error()
    rc = lib.pccnn_compute_pdf_grid(3, None, None, None, 10, None, None, 4, None, 0, None, None, 2, 300, None, None, None)
    assert rc == -2 and b"d=2" in lib.pccnn_last_error()
    assert lib.pccnn_compute_pdf_grid(3, None, None, None, 0, None, None, 4, None, 0, None, None, 3, 300, None, None,
                                      None) == 0
    assert lib.pccnn_grid_build_workspace_bytes(1000) == lib.pccnn_sort_keys_workspace_bytes(1000)
    assert lib.pccnn_conv_workspace_bytes(1000, 5000, 32, 16, 64, 0) >= 1000 * 32 * 16 * 4
    assert lib.pccnn_find_neighbors_workspace_bytes(500, 1000) >= 4000 + 500 * 16


def test_op_module_exports_reference_names():
    from pccnn_lib_amd import pccnn_lib_ops
    assert len(pccnn_lib_ops.REFERENCE_NAMES) == 26
    for name in pccnn_lib_ops.REFERENCE_NAMES:
        assert callable(getattr(pccnn_lib_ops, name))
    # every family validates its tensors before touching the library
    import torch
    z = torch.zeros(4, 3)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        pccnn_lib_ops.sph_conv(z, z, z, z, z, z, z, z, z, z)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        pccnn_lib_ops.point_conv(z, z, z, z, z)


def test_ops_reject_cpu_tensors():
    import torch
    from pccnn_lib_amd import pccnn_lib_ops
    with pytest.raises(RuntimeError, match="GPU tensor"):
        pccnn_lib_ops.compute_keys(torch.zeros(4, 3), torch.zeros(4, dtype=torch.int32), torch.zeros(1, 3),
                                   torch.ones(3, dtype=torch.int32), torch.ones(3))


def test_layers_keep_reference_parameter_names():
    from pccnn_lib_amd.pc.layers import KPConv, MCConv
    kp = KPConv(3, 8, 16, 15)
    assert set(kp.state_dict()) == {"kernel_pts_", "sigma_", "conv_weights_"}
    assert tuple(kp.conv_weights_.shape) == (15 * 8, 16) and tuple(kp.kernel_pts_.shape) == (15, 3)
    assert abs(float(kp.kernel_pts_[0].abs().sum())) == 0.0 and 0 < float(kp.sigma_) < 1
    mc = MCConv(3, 8, 16, 16, 2)
    assert set(mc.state_dict()) == {"proj_axis_", "proj_bias_", "conv_weights_"}
    assert tuple(mc.conv_weights_.shape) == (2, 16 * 8, 8) and tuple(mc.proj_axis_.shape) == (3, 32)
    from pccnn_lib_amd.pc.layers import KPConvN, PCCNN, PointConv, SPHConv
    for cls, scale in ((KPConvN, 2.0), (PCCNN, 0.4)):
        layer = cls(3, 8, 16, 16)
        assert set(layer.state_dict()) == {"kernel_pts_", "sigma_", "conv_weights_"}
        assert abs(float(layer.sigma_) / float(KPConv(3, 8, 16, 16).sigma_) - scale) < 1e-6
    sph = SPHConv(3, 8, 16, 2, 5, 3)
    assert set(sph.state_dict()) == {"radial_bins_", "azimuz_bins_", "polar_bins_", "conv_weights_"}
    assert tuple(sph.conv_weights_.shape) == (31 * 8, 16)
    pcv = PointConv(3, 8, 16, 16)
    assert {"proj_axis_", "proj_bias_", "conv_weights_", "pdf_mlp_.0.weight", "pdf_mlp_.2.weight"} <= set(pcv.state_dict())


def test_kernel_point_layers_hold_the_reference_buffers():
    """kernel_pts_ / sigma_ of a new layer, for every constant layout of the reference, against the fixture that
    applies pccnn_lib/pc/layers/KPConv.py:46-57 to the reference's tables (tests/golden/make_kernel_point_buffers.py)."""
    import torch
    from pccnn_lib_amd.pc.layers import KPConv, KPConvN, PCCNN
    from pccnn_lib_amd.pc.layers.kernel_points import kernel_pts_dict, load_tables
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kernel_point_buffers.npz"))
    keys = sorted(k[len("table_"):] for k in gold.files if k.startswith("table_"))
    assert keys == sorted(load_tables()) and len(keys) == 12
    for key in keys:
        dims, count = (int(v) for v in key.split("_"))
        assert np.array_equal(kernel_pts_dict[key], gold["table_" + key]), key
        layer = KPConv(dims, 4, 4, count)
        assert layer.kernel_pts_.dtype == torch.float32 and layer.sigma_.dtype == torch.float32
        assert np.array_equal(layer.kernel_pts_.numpy(), gold["kernel_pts_" + key]), key
        assert float(layer.sigma_) == float(gold["sigma_" + key]), key
    # KPConvN and PCCNN scale sigma by 2 and 0.4 (KPConvN.py:57, PCCNN.py:57); their rotation is seeded with the
    # clock (KPConvN.py:53, PCCNN.py:53), so only what a rotation keeps is compared: norms and mutual distances
    for cls, scale in ((KPConvN, 2.0), (PCCNN, 0.4)):
        layer = cls(3, 4, 4, 16)
        got, exp = layer.kernel_pts_.numpy().astype(np.float64), gold["kernel_pts_3_16"].astype(np.float64)
        assert np.allclose(got @ got.T, exp @ exp.T, atol=1e-6)
        d = float(gold["sigma_3_16"]) / (1.0 - float(gold["sigma_3_16"]))
        assert abs(float(layer.sigma_) - scale * d / (1.0 + d)) < 1e-6


def test_model_base_class_drives_the_layers_initialisation():
    # pccnn_lib/pc/models/IModel.py:6-27: the layers are kept in order, the warm-up switch reaches the layer, and
    # init_variance redraws the weights with variance out_constant_variance / (divisor * input features)
    import torch
    import pccnn_lib_amd as lib
    model = lib.pc.models.IModel()
    assert lib.pc.IModel is lib.pc.models.IModel and model.get_num_convs() == 0
    torch.manual_seed(0)
    kp = lib.pc.layers.KPConv(3, 64, 32, 16, True, 2.0)
    point = lib.pc.layers.PointConv(3, 32, 16, 8, True, 1.0)
    model.add_conv(kp)
    model.add_conv(point)
    assert model.get_num_convs() == 2 and model.conv_list_[1] is point
    model.set_init_warmup_state(0, True)
    assert kp.wamup_state_ is True and point.wamup_state_ is False
    model.init_variance(0, 4.0)
    want = 2.0 / (4.0 * 64)
    assert abs(float(kp.conv_weights_.detach().var()) - want) < 0.05 * want
    assert point.init_proj_axis_ is False
    model.init_variance(1, 1.0)
    want = 1.0 / 32
    assert abs(float(point.conv_weights_.detach().var()) - want) < 0.1 * want
    assert point.init_proj_axis_ is True            # a PointConv layer redraws its axes on the next warm-up pass


def test_torch_functions_apply_to_a_clouds_coordinates():
    # pccnn_lib/pc/Pointcloud.py:158-165
    import torch
    import pccnn_lib_amd as lib
    pts = torch.arange(12, dtype=torch.float32).reshape(4, 3)
    ids = torch.tensor([0, 0, 1, 1], dtype=torch.int32)
    cloud = lib.pc.Pointcloud(pts, ids)
    moved = torch.add(cloud, 1.5)
    assert isinstance(moved, lib.pc.Pointcloud) and torch.equal(moved.pts_, pts + 1.5)
    assert moved.batch_ids_ is cloud.batch_ids_ and int(moved.batch_size_) == 2
    scaled = torch.mul(cloud, torch.tensor([2.0, 1.0, 0.5]))
    assert torch.equal(scaled.pts_, pts * torch.tensor([2.0, 1.0, 0.5]))
    both = torch.sub(moved, cloud)
    assert torch.equal(both.pts_, torch.full((4, 3), 1.5))


def test_install_as_reference_resolves_the_reference_imports():
    # in a process of its own: the call registers modules under the reference's names
    import subprocess
    import sys
    code = ("import pccnn_lib_amd; pccnn_lib_amd.install_as_reference()\n"
            "import pccnn_lib, pccnn_lib_ops\n"
            "from pccnn_lib.pc import Pointcloud, BoundingBox, Grid, Neighborhood, PointPooling\n"
            "from pccnn_lib.pc.layers import KPConv, MCConv, KPConvN, PCCNN, PointConv, SPHConv\n"
            "from pccnn_lib.op_wrappers import ComputeKeys, BuildGridDS, FindNeighbors, ComputePDF\n"
            "assert pccnn_lib.pc.Pointcloud is pccnn_lib_amd.pc.Pointcloud\n"
            "assert callable(pccnn_lib_ops.compute_keys) and callable(pccnn_lib_ops.mc_conv_grads)\n")
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr


def test_the_op_module_imports_under_the_reference_name():
    """`import pccnn_lib_ops` alone, in a fresh process, as pccnn_lib/op_wrappers/*.py do."""
    import subprocess
    import sys
    code = ("import pccnn_lib_ops\n"
            "assert len(pccnn_lib_ops.REFERENCE_NAMES) == 26\n"
            "assert all(callable(getattr(pccnn_lib_ops, n)) for n in pccnn_lib_ops.REFERENCE_NAMES)\n")
    res = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr


def test_point_side_keeps_the_plain_route_unless_the_pairs_are_in_key_order():
    # host logic of the layers (no GPU): a convolution reads the cloud's own tensors and the reference's pair list
    # unless its neighborhood kept the pairs in key order, belongs to this cloud, and no gradient goes to the positions
    import types
    import torch
    from pccnn_lib_amd.pc.layers import conv_base
    feats = torch.ones(4, 2)
    cloud = types.SimpleNamespace(pts_=torch.zeros(4, 3))
    plain = types.SimpleNamespace(neighbors_key_order_=None, neighbors_=torch.zeros(2, 2, dtype=torch.int32),
                                  grid_=types.SimpleNamespace(pointcloud_=cloud))
    pts, pairs, moved = conv_base.point_side(cloud, plain, feats)
    assert pts is cloud.pts_ and pairs is plain.neighbors_ and moved is feats
    other = types.SimpleNamespace(pts_=torch.zeros(4, 3))
    keyed = types.SimpleNamespace(neighbors_key_order_=torch.ones(2, 2, dtype=torch.int32),
                                  neighbors_=torch.zeros(2, 2, dtype=torch.int32),
                                  grid_=types.SimpleNamespace(pointcloud_=other))
    pts, pairs, moved = conv_base.point_side(cloud, keyed, feats)             # a neighborhood of another cloud
    assert pts is cloud.pts_ and pairs is keyed.neighbors_ and moved is feats
    wanted = types.SimpleNamespace(pts_=torch.zeros(4, 3, requires_grad=True))
    keyed.grid_.pointcloud_ = wanted
    pts, pairs, moved = conv_base.point_side(wanted, keyed, feats)            # positions that want a gradient
    assert pts is wanted.pts_ and pairs is keyed.neighbors_ and moved is feats
    layer = conv_base.IConvLayer(3, 2, 2)
    assert layer.key_order_capable_ is False and conv_base.KEY_ORDER_MIN_POINTS >= 100000


@pytest.fixture(scope="module")
def compiled_module(lib_path):
    from pccnn_lib_amd import build
    if not os.path.exists(build.extension_path()):
        build.build_extension(verbose=False)
    from pccnn_lib_amd import pccnn_lib_ops as ops
    before = ops.use_binding("compiled")
    ops.use_binding(before)
    import sys
    return sys.modules["pccnn_lib_ops"]


def test_import_of_the_reference_name_resolves_to_the_compiled_extension(compiled_module):
    # setup.py:7-8 of the reference builds an extension module named pccnn_lib_ops; so does this build, and a plain
    # `import pccnn_lib_ops` from the repository root finds the shared object rather than the Python stand-in
    import subprocess
    import sys
    code = ("import pccnn_lib_ops as m\n"
            "assert m.__file__.endswith('.so'), m.__file__\n"
            "assert m.binding == 'compiled' and len(m.REFERENCE_NAMES) == 26\n"
            "assert all(callable(getattr(m, n)) for n in m.REFERENCE_NAMES)\n")
    res = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr


@pytest.mark.parametrize("which", ["compiled", "ctypes"])
def test_both_bindings_export_the_reference_names_and_validate_on_the_host(compiled_module, which):
    import torch
    from pccnn_lib_amd import pccnn_lib_ops as ops
    before = ops.use_binding(which)
    try:
        assert ops.binding == which
        for name in ops.REFERENCE_NAMES:
            assert callable(getattr(ops, name)) and getattr(ops, name) is ops.BINDINGS[which][name]
        z, zi = torch.zeros(4, 3), torch.zeros(4, dtype=torch.int32)
        with pytest.raises(RuntimeError, match="GPU tensor"):
            ops.compute_keys(z, zi, torch.zeros(1, 3), torch.ones(3, dtype=torch.int32), torch.ones(3))
        with pytest.raises(RuntimeError, match="GPU tensor"):
            ops.sph_conv(z, z, z, z, z, z, z, z, z, z)
        with pytest.raises(RuntimeError, match="GPU tensor"):
            ops.point_conv(z, z, z, z, z)
        with pytest.raises(RuntimeError, match="GPU tensor"):
            ops.mc_conv_grads(z, z, z, z, z, z, z, z, z, z, z, grad_mask=ops.GRAD_FEATS, contraction="bf16")
    finally:
        ops.use_binding(before)


def test_compiled_functions_take_the_arguments_of_the_ctypes_functions(compiled_module):
    # same parameter count and the same keyword additions (return_proj, proj, grad_mask, mirror, contraction), read
    # from the signature line pybind11 writes into each docstring
    import inspect
    from pccnn_lib_amd import pccnn_lib_ops as ops
    for name in ops.REFERENCE_NAMES:
        py_params = list(inspect.signature(ops.BINDINGS["ctypes"][name]).parameters.values())
        line = getattr(compiled_module, name).__doc__.splitlines()[0]
        inner = line[line.index("(") + 1:line.rindex(")")]
        c_params = [p for p in re.split(r",\s*(?![^\[]*\])", inner) if p]
        assert len(c_params) == len(py_params), (name, line)
        for cp, pp in zip(c_params, py_params):
            if pp.default is not inspect.Parameter.empty:
                assert cp.split(":")[0].strip() == pp.name and "=" in cp, (name, cp, pp.name)
