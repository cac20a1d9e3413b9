"""CPU-only tests: the C-ABI library loads and exports every declared symbol,
argument validation happens before any GPU work, and the host-side mirror of the
reference API has the reference's names, defaults and parameter layout."""
import ctypes

import numpy as np
import pytest
import torch

from rfa_amd import _lib


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _lib.declared_symbols()
    assert len(declared) >= 19
    for name in declared:
        assert hasattr(lib, name), name
    assert set(declared) == set(_lib.SIGNATURES)
    assert lib.rfa_version() >= 100


def test_shape_support_and_workspace_queries():
    lib = _lib.load()
    assert lib.rfa_shape_supported(128, 64) == 1 and lib.rfa_shape_supported(256, 128) == 1
    assert lib.rfa_shape_supported(100, 64) == 0 and lib.rfa_shape_supported(128, 48) == 0
    assert lib.rfa_feature_map_supported(64, 64) == 1 and lib.rfa_feature_map_supported(48, 64) == 0
    assert lib.rfa_causal_num_segments(1024, 64, 128, 64) >= 1
    assert lib.rfa_causal_num_segments(64, 1, 128, 64) == 1          # one chunk cannot be split
    assert lib.rfa_causal_forward_workspace_bytes(0, 4, 128, 64) == 0
    fw = lib.rfa_causal_forward_workspace_bytes(1024, 64, 128, 64)
    bw = lib.rfa_causal_backward_workspace_bytes(1024, 64, 128, 64)
    assert bw > fw >= 0 and bw >= 2 * 1024 * 64 * 4
    assert lib.rfa_feature_map_backward_workspace_bytes(8192, 8, 64, 64) >= 8 * 64 * 64 * 4


def test_tuning_knobs_round_trip():
    lib = _lib.load()
    assert _lib.tuning_get("nseg") == -1
    with _lib.tuning(nseg=3, prefix=1):
        assert _lib.tuning_get("nseg") == 3 and _lib.tuning_get("prefix") == 1
        assert lib.rfa_causal_num_segments(1024, 64, 128, 64) == 3
    assert _lib.tuning_get("nseg") == -1 and _lib.tuning_get("prefix") == -1
    with pytest.raises(_lib.RfaHipError, match="no knob"):
        _lib.tuning_set("no_such_knob", 1)
    # the saved buffer grows by its 256-byte header and follows the plan
    with _lib.tuning(nseg=1, sliced=0):
        one = lib.rfa_causal_saved_state_bytes(1024, 64, 128, 64)
    with _lib.tuning(nseg=4, prefix=0, sliced=0):
        four = lib.rfa_causal_saved_state_bytes(1024, 64, 128, 64)
    assert one >= 256 + 64 * (128 * 64 + 128) * 4 + 1024 * 64 * 4 and four >= one + 3 * 64 * 128 * 64 * 4
    # with the final-state layout the buffer holds one state per sequence whatever the segment count
    with _lib.tuning(nseg=4, sliced=1):
        assert lib.rfa_causal_saved_state_bytes(1024, 64, 128, 64) == one


def test_errors_are_reported_before_any_gpu_work():
    lib = _lib.load()
    rc = lib.rfa_causal_forward(None, None, None, None, 16, 2, 100, 64, None, 0, None)
    assert rc == -3 and b"K=100" in lib.rfa_last_error()
    rc = lib.rfa_causal_forward(None, None, None, None, 16, 2, 128, 64, None, 0, None)
    assert rc == -1
    rc = lib.rfa_causal_forward(None, None, None, None, -1, 2, 128, 64, None, 0, None)
    assert rc == -2
    buf = ctypes.create_string_buffer(64)
    odd = ctypes.addressof(buf) + 1
    rc = lib.rfa_causal_forward(odd, odd, odd, odd, 16, 2, 128, 64, None, 0, None)
    assert rc == -4
    al = (ctypes.addressof(buf) + 15) & ~15
    rc = lib.rfa_causal_backward(al, al, al, al, al, al, al, 16, 2, 128, 64, None, 0, None)
    assert rc == -5 and b"workspace" in lib.rfa_last_error()
    assert lib.rfa_causal_forward(None, None, None, None, 0, 2, 128, 64, None, 0, None) == 0   # empty input
    assert lib.rfa_feature_map_forward(None, None, None, 4, 2, 48, 64, 0.1, None) == -3
    assert lib.rfa_incremental(None, None, None, None, None, None, 1, 2, 128, 64, None) == -1
    with pytest.raises(_lib.RfaHipError):
        _lib.check(-3)


@pytest.mark.usefixtures("binding")
def test_host_wrappers_reject_cpu_and_wrong_dtype():
    from rfa_amd import RFA, rfa_hip
    q = torch.zeros(4, 2, 128, dtype=torch.float16)
    v = torch.zeros(4, 2, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        rfa_hip.forward(q, q, v)
    with pytest.raises(RuntimeError, match="no CPU path"):
        RFA.apply(q, q, v)
    with pytest.raises(RuntimeError):
        rfa_hip.feature_map_forward(torch.zeros(2, 1, 2, 64, dtype=torch.float16), torch.zeros(2, 64, 64, dtype=torch.float16), 0.1)


def test_formula_statements_match_oracle_on_cpu():
    """RFA.forward_torch / backward_torch / reverse_cumsum are kept as API; they are
    plain formulas and must agree with the oracle."""
    from oracle import rfa_oracle as O
    from rfa_amd.rfa import RFA, reverse_cumsum, rfa_debug
    g = torch.Generator().manual_seed(0)
    q, k = (0.1 * torch.randn(9, 2, 8, generator=g, dtype=torch.float64) for _ in range(2))
    k = k.abs()
    v, go = (torch.randn(9, 2, 4, generator=g, dtype=torch.float64) for _ in range(2))
    assert torch.allclose(RFA.forward_torch(q, k, v), O.causal_forward_loop(q, k, v)[0], atol=1e-12)
    assert torch.allclose(rfa_debug(q, k, v), O.causal_forward_quadratic(q, k, v), atol=1e-12)
    for a, b in zip(RFA.backward_torch(q, k, v, go), O.causal_backward_chunked(q, k, v, go, chunk=4)):
        assert torch.allclose(a, b, atol=1e-11)
    x = torch.arange(6.0).reshape(3, 2)
    assert torch.equal(reverse_cumsum(x, 0), torch.tensor([[6.0, 9.0], [6.0, 8.0], [4.0, 5.0]]))


def test_module_parameter_names_and_defaults():
    from rfa_amd import CausalAttention, CrossAttention, CrossAttentionProject, CrossAttentionState
    from rfa_amd.utils import EPS, SCALE
    assert EPS == 1.0 and SCALE == 0.1
    m = CausalAttention(embed_dim=128, num_heads=2, head_dim=64, proj_dim=64)
    assert sorted(m.state_dict()) == sorted(
        [f"{p}.{w}" for p in ("q_proj", "k_proj", "v_proj", "out_proj") for w in ("weight", "bias")] + ["sigma"])
    assert tuple(m.sigma.shape) == (2, 1, 64) and torch.all(m.sigma == 1) and torch.all(m.out_proj.bias == 0)
    assert m.tau == 1.0 and m.reparam_proj and m.cuda_causal_rfa and callable(m.upgrade_state_dict_named)
    assert "sigma" not in CausalAttention(embed_dim=128, num_heads=2, head_dim=64, proj_dim=64,
                                          reparam_proj=False).state_dict()
    c = CrossAttention(embed_dim=128, num_heads=2, head_dim=64, proj_dim=64)
    assert sorted(c.state_dict()) == ["out_proj.bias", "out_proj.weight", "q_proj.bias", "q_proj.weight"]
    assert torch.all(c.q_proj.bias == 0)
    p = CrossAttentionProject(num_layers=3, embed_dim=128, num_heads=2, head_dim=64, proj_dim=32)
    keys = set(p.state_dict())
    assert {"layers.0.k_proj.weight", "layers.2.v_proj.bias", "layers.1.sigma", "random_matrices",
            "random_matrices_eval"} <= keys
    assert tuple(p.random_matrices.shape) == (500, 32, 64) and p.random_matrices.dtype == torch.float16
    assert tuple(p.random_matrices_eval.shape) == (2, 32, 64) and not p.random_matrices_eval.requires_grad
    assert CrossAttentionState._fields == ("s", "z", "random_matrices", "tau")


def test_sample_and_build_random_matrices():
    from rfa_amd.utils import build_random_matrices, sample_random_matrices
    mats = torch.arange(20 * 2 * 3, dtype=torch.float32).reshape(20, 2, 3)
    np.random.seed(0)
    per_layer = sample_random_matrices(num_layers=3, num_heads=4, random_matrices=mats, is_training=True)
    assert len(per_layer) == 3 and all(tuple(m.shape) == (4, 2, 3) for m in per_layer)
    firsts = torch.cat(per_layer)[:, 0, 0]
    assert len(set(firsts.tolist())) == 12                    # drawn without replacement
    assert torch.equal(sample_random_matrices(num_layers=3, num_heads=4, random_matrices=mats, is_training=False), mats[:4])
    W = torch.ones(2, 3, 4)
    sigma = torch.tensor([[[1.0, 2.0, 3.0, 4.0]], [[5.0, 6.0, 7.0, 8.0]]])
    out = build_random_matrices(W, 2.0, sigma, True)
    assert torch.equal(out[1, 2], torch.tensor([2.5, 3.0, 3.5, 4.0]))
    assert torch.equal(build_random_matrices(W, 4.0), W / 4.0)


def test_load_random_matrices_leaves_the_global_numpy_generator_alone():
    """The matrix file does not ship, so every CrossAttentionProject generates the matrices in
    memory; that must not reseed numpy for the caller (sample_random_matrices and any numpy-based
    shuffling draw from the global generator afterwards)."""
    from rfa_amd.construct_random_matrices import construct_random_matrices, rrf
    from rfa_amd.utils import load_random_matrices
    draws = []
    for seed in (7, 99):
        np.random.seed(seed)
        mats = load_random_matrices(head_dim=64, proj_dim=32)
        draws.append(np.random.rand())
    assert draws[0] != draws[1]
    np.random.seed(7)
    assert draws[0] == np.random.rand()
    want = construct_random_matrices(rrf, 500, head_dim=64, proj_dim=32, seed=31415)   # the reference script's recipe
    assert torch.equal(mats, torch.tensor(want, dtype=torch.half))


def test_masked_rfa_has_no_cpu_path():
    """masked_rfa runs on the quadratic-form HIP kernels only: CPU tensors raise."""
    from rfa_amd.causal_attention import masked_rfa
    pq = torch.rand(4, 1, 1, 64).half()
    v = torch.rand(4, 1, 1, 64).half()
    with pytest.raises((RuntimeError, ImportError)):
        masked_rfa(phi_q=pq, phi_k=pq, v=v)


def test_random_matrix_generators():
    from rfa_amd.construct_random_matrices import construct_random_matrices, orf, rrf, softmax_kernel_error
    a = construct_random_matrices(rrf, 3, head_dim=8, proj_dim=16, seed=31415)
    b = construct_random_matrices(rrf, 3, head_dim=8, proj_dim=16, seed=31415)
    assert a.shape == (3, 16, 8) and np.array_equal(a, b)
    # a generator handed in: same stream as the seeded global one, global state untouched
    np.random.seed(7)
    before = np.random.get_state()[1].copy()
    c = construct_random_matrices(rrf, 3, head_dim=8, proj_dim=16, rng=np.random.RandomState(31415))
    assert np.array_equal(a, c) and np.array_equal(np.random.get_state()[1], before)
    np.random.seed(1)
    o = orf(head_dim=16, proj_dim=16)
    unit = o / np.linalg.norm(o, axis=1, keepdims=True)
    assert np.allclose(unit @ unit.T, np.eye(16), atol=1e-10)      # orthogonal directions
    np.random.seed(2)
    assert softmax_kernel_error(16, 2048, rrf(head_dim=16, proj_dim=2048), iters=5) < 0.15


def test_both_bindings_expose_the_same_functions():
    """The torch extension and the ctypes wrappers stand behind one set of names."""
    from rfa_amd import rfa_hip
    assert rfa_hip.ext_available(), "python -m rfa_amd.build builds the torch binding"
    before = rfa_hip.binding()
    try:
        for name in ("ext", "ctypes"):
            rfa_hip.use_binding(name)
            assert rfa_hip.binding() == name
            for fn in rfa_hip._BOUND:
                assert callable(getattr(rfa_hip, fn)), (name, fn)
            assert rfa_hip.supported(128, 64) and not rfa_hip.supported(100, 64)
        with pytest.raises(ValueError):
            rfa_hip.use_binding("pybind")
    finally:
        rfa_hip.use_binding(before)
    assert before == "ext"          # the default when the extension is there


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """No fallback of any kind: without the built library the first call raises ImportError that
    says how to build it, and the ctypes table binds every declared entry point (a signature
    missing there would only show up when that entry point is first called)."""
    from rfa_amd import _lib
    assert sorted(_lib.SIGNATURES) == sorted(s for s in _lib.declared_symbols() if s != "rfa_debug_phase_ticks")
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "librfa_hip.so"))
    with pytest.raises(ImportError, match="rfa_amd.build"):
        _lib.load()


def test_binding_built_after_the_package_was_imported_is_found(tmp_path):
    """A clean tree has no _rfa_hip_ext.so when the package is first imported (the build entry point
    imports the package to reach the build recipe).  Once the file is there, ext_available() and
    use_binding('ext') must find it in the same process."""
    import os
    import shutil
    import subprocess
    import sys
    from rfa_amd import build as B
    if not (os.path.exists(B.EXT_PATH) and os.path.exists(B.LIB_PATH)):
        pytest.skip("the torch binding has not been built")
    pkg = tmp_path / "rfa_amd"
    shutil.copytree(os.path.dirname(B.__file__), pkg,
                    ignore=shutil.ignore_patterns("_rfa_hip_ext*.so", "__pycache__", "csrc"))
    code = (
        "import os, shutil, sys\n"
        f"sys.path.insert(0, {str(tmp_path)!r})\n"
        "os.environ.pop('RFA_AMD_BINDING', None)\n"
        "import rfa_amd\n"
        "from rfa_amd import rfa_hip\n"
        f"assert rfa_amd.__file__.startswith({str(tmp_path)!r})\n"
        "assert not rfa_hip.ext_available() and rfa_hip.binding() == 'ctypes'\n"
        f"shutil.copy({B.EXT_PATH!r}, os.path.dirname(rfa_amd.__file__))\n"
        "assert rfa_hip.ext_available()\n"
        "rfa_hip.use_binding('ext')\n"
        "assert rfa_hip.binding() == 'ext' and rfa_hip.forward.__module__.endswith('_rfa_hip_ext')\n"
        "print('found')\n")
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=str(tmp_path))
    assert proc.returncode == 0 and "found" in proc.stdout, proc.stdout + proc.stderr


def test_derived_values_answer_only_for_the_same_live_tensors_in_the_same_state():
    """The keep-until-changed store behind the stacked projection weights and the scaled random
    matrices: a hit needs the same tensor objects with unchanged version, address, dtype and shape;
    a tensor that died cannot be stood in for by another one, whatever address or id it got."""
    import gc
    from rfa_amd._derived import derived
    slot, made = {}, []

    def make_from(*ts):
        def make():
            made.append(1)
            return sum(float(t.sum()) for t in ts if t is not None)
        return make

    a, b = torch.ones(4), torch.full((4,), 2.0)
    assert derived(slot, "k", (a, b, None), 1, make_from(a, b)) == 12.0 and len(made) == 1
    assert derived(slot, "k", (a, b, None), 1, make_from(a, b)) == 12.0 and len(made) == 1      # hit
    assert derived(slot, "k", (a, b, None), 2, make_from(a, b)) == 12.0 and len(made) == 2      # other extra
    a.add_(1.0)                                                                                   # version moves
    assert derived(slot, "k", (a, b, None), 2, make_from(a, b)) == 16.0 and len(made) == 3
    a.data = torch.zeros(4)                                                                       # address moves, version does not
    assert derived(slot, "k", (a, b, None), 2, make_from(a, b)) == 8.0 and len(made) == 4
    c = b.clone()                                                                                 # equal state, another object
    assert derived(slot, "k", (a, c, None), 2, make_from(a, c)) == 8.0 and len(made) == 5
    assert derived(slot, "k", (a, None, None), 2, make_from(a)) == 0.0 and len(made) == 6       # None where a tensor was
    # a dead source: the entry must not answer for a newcomer in the same state, even at the same address
    t = torch.full((1024,), 3.0)
    derived(slot, "dead", (t,), None, make_from(t))
    n_made, ptr = len(made), t.data_ptr()
    del t
    gc.collect()
    for _ in range(8):
        u = torch.full((1024,), 5.0)
        if u.data_ptr() == ptr:
            break
    assert derived(slot, "dead", (u,), None, make_from(u)) == 5.0 * 1024 and len(made) == n_made + 1
    # bounded slots drop entries of dead sources first
    small = {}
    keep = [torch.ones(2) for _ in range(3)]
    for i, t in enumerate(keep):
        derived(small, i, (t,), None, make_from(t), limit=3)
    del keep[0]
    gc.collect()
    extra = torch.ones(2)
    derived(small, "new", (extra,), None, make_from(extra), limit=3)
    assert set(small) == {1, 2, "new"}
