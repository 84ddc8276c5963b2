"""CPU-side checks: the C-ABI library loads and exports what the header declares, and the host logic
(geometry, synthetic batches, parameter plumbing, error behaviour) works without a GPU."""
import ctypes
import os
import re

import pytest
import torch

from crystalframer_amd import _lib, cuda_funcs, geometry, params, synthetic
from oracle import torch_oracle as TO

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "crystalframer_hip.h")).read()
    declared = set(re.findall(r"\b(cfh_[a-z0-9_]+)\s*\(", header))
    assert {"cfh_frame_axis1", "cfh_frame_axis2", "cfh_framed_pe_forward", "cfh_framed_pe_backward",
            "cfh_workspace_bytes", "cfh_last_error", "cfh_abi_version"} <= declared
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert set(_lib.EXPORTS) == declared
    assert lib.cfh_abi_version() == _lib.ABI_VERSION


def test_params_struct_matches_header_layout():
    header = open(os.path.join(ROOT, "include", "crystalframer_hip.h")).read()
    body = header[header.index("typedef struct cfh_params"):header.index("} cfh_params;")]
    fields = re.findall(r"^\s*(?:int32_t|float|uint64_t|uint64_t\*)\s+([a-z0-9_]+);", body, flags=re.M)
    assert fields == [f[0] for f in _lib.CfhParams._fields_]
    assert ctypes.sizeof(_lib.CfhParams) == 104


def test_argument_errors_are_reported_without_a_gpu():
    lib = _lib.load()
    p = cuda_funcs._params(8, 16, 64, 64, 0, 14.0, 1.0, 4.0, 1.0, 1.0, -3.5)
    p.head_dim = 32
    assert lib.cfh_workspace_bytes(ctypes.byref(p), 10, 100) == 0
    assert b"head_dim" in lib.cfh_last_error()
    p.head_dim = 16
    p.struct_size = 4
    rc = lib.cfh_framed_pe_forward(ctypes.byref(p), *([None] * 13), 1, 1, 1, None, None, None, None, None, 0, None)
    assert rc == -1 and b"struct_size" in lib.cfh_last_error()


def test_operators_refuse_cpu_tensors():
    a = torch.zeros(2, 8)
    with pytest.raises(RuntimeError, match="HIP device"):
        cuda_funcs.RealEncodingWithFramedProjFuncCUDA.apply(
            a, torch.zeros(4, 3), None, torch.eye(3)[None], torch.zeros(2, dtype=torch.long),
            torch.zeros(2, 4, dtype=torch.long), 0, 14.0, 1.0, None, None, None, None, None, None, None,
            0, 4.0, 0, 1.0, 1.0)


def test_compile_kernels_validates_constants():
    cuda_funcs.compile_kernels(2, 8, 16, 64, 64, 16, True, 0, 1.0, 4.0, 1.0, 1.0, 1e-5)
    assert cuda_funcs.KernelManager.LATTICE_RANGE == 2 and cuda_funcs.KernelManager.MINIMUM_RANGE == 2
    cuda_funcs.compile_kernels(3, 8, 16, 64, 0, 16, False, 1, 1.0, 4.0, 1.0, 1.0, 0.0)
    assert cuda_funcs.KernelManager.LATTICE_RANGE == 3 and cuda_funcs.KernelManager.MINIMUM_RANGE == 0
    with pytest.raises(NotImplementedError):
        cuda_funcs.compile_kernels(2, 8, 32, 64, 64, 32, True, 0, 1.0, 4.0, 1.0, 1.0, 1e-5)
    # the 16-bin angle basis of the lightweight setting (train_jarvis_time.sh:40-57) and the default's scale with it
    cuda_funcs.compile_kernels(2, 8, 16, 64, 16, 16, True, 0, 1.0, 1.0, 1.5, 6.0, 1e-5)
    cuda_funcs.compile_kernels(2, 8, 16, 64, 16, 16, True, 1, 1.0, 4.0, 1.0, 1.0, 1e-5)
    with pytest.raises(NotImplementedError):
        cuda_funcs.compile_kernels(2, 8, 16, 64, 32, 16, True, 0, 1.0, 4.0, 1.0, 1.0, 1e-5)      # 32 angle bins
    with pytest.raises(NotImplementedError):
        cuda_funcs.compile_kernels(2, 8, 16, 64, 64, 16, True, 0, 1.0, 1.0, 1.0, 1.0, 1e-5)      # 64 bins, scale 1
    with pytest.raises(NotImplementedError):
        cuda_funcs.compile_kernels(2, 8, 16, 64, 16, 16, True, 0, 1.0, 0.5, 1.0, 1.0, 1e-5)      # 16 bins, scale < 1
    cuda_funcs.compile_kernels(2, 8, 16, 64, 64, 16, True, 0, 1.0, 4.0, 1.0, 1.0, 1e-5)


def test_geometry_matches_oracle_geometry():
    cb = synthetic.make_config("C1", seed=5)
    geo = geometry.crystal_geometry(cb.pos, cb.batch, cb.trans_vec, cb.sizes)
    edges, rpos, recip, vcell = TO.geometry(cb.pos.double(), cb.trans_vec.double(), cb.sizes.tolist())
    assert torch.equal(geo.edges, edges)
    assert (geo.rpos.double() - rpos).abs().max() < 1e-5
    assert (geo.recip.double() - recip).abs().max() < 1e-5
    assert (geo.rvlen.double() - recip.norm(dim=-1)).abs().max() < 1e-5
    assert (geo.vcell.double() - vcell).abs().max() < 1e-3
    n = cb.sizes[cb.batch]
    assert torch.equal(geo.e_start[1:] - geo.e_start[:-1], n)
    assert torch.equal(geo.e_start, cuda_funcs.edge_schedule(geo.edges, cb.pos.shape[0])[0])
    assert sorted(geo.order.tolist()) == list(range(cb.pos.shape[0]))
    assert (n[geo.order.long()][:-1] >= n[geo.order.long()][1:]).all()
    # reciprocal rows are dual to the lattice rows: b_i . t_j = 2 pi delta_ij
    dual = torch.einsum("bix,bjx->bij", geo.recip.double(), cb.trans_vec.double())
    assert (dual - 2 * torch.pi * torch.eye(3, dtype=torch.float64)).abs().max() < 1e-4


@pytest.mark.parametrize("name", ["C1", "C2", "C4", "C5"])
def test_synthetic_configs_have_the_documented_shape(name):
    cb = synthetic.make_config(name, seed=123, num_crystals=64 if name == "C5" else None)
    spec = synthetic.CONFIGS[name]
    assert cb.sizes.min() >= spec["atoms_lo"] and cb.sizes.max() <= spec["atoms_hi"]
    lengths = cb.trans_vec.norm(dim=-1)
    assert lengths.min() >= spec["len_lo"] - 1e-4 and lengths.max() <= spec["len_hi"] + 1e-4
    assert (cb.x.sum(-1) == 1).all() and cb.x.shape[1] == 98
    assert geometry.det_3x3(cb.trans_vec).min() > 0
    again = synthetic.make_config(name, seed=123, num_crystals=64 if name == "C5" else None)
    assert torch.equal(cb.pos, again.pos) and torch.equal(cb.sizes, again.sizes)
    frac = torch.linalg.solve(cb.trans_vec[cb.batch].transpose(1, 2).double(), cb.pos.double().unsqueeze(-1)).squeeze(-1)
    assert frac.min() > -1e-4 and frac.max() < 1 + 1e-4


def test_model_has_reference_parameter_names_and_count():
    from crystalframer_amd import latticeformer
    m = latticeformer.Latticeformer(params.ModelParams())
    sd = m.state_dict()
    for key, shape in [("input_embeddings.weight", (128, 98)),
                       ("encoder.layers.0.self_attn.q_proj_weight", (128, 128)),
                       ("encoder.layers.3.self_attn.pe_dist_proj", (1, 8, 16, 64)),
                       ("encoder.layers.2.self_attn.proj_angle3", (1, 8, 16, 64)),
                       ("encoder.layers.1.self_attn.lattice_pos_weights", (128,)),
                       ("encoder.layers.1.self_attn.gauss_scale", (2,)),
                       ("encoder.layers.0.self_attn.in_proj_bias", (384,)),
                       ("encoder.layers.0.self_attn.out_proj.weight", (128, 128)),
                       ("encoder.layers.0.linear1.weight", (512, 128)),
                       ("mlp.0.weight", (128, 128)), ("mlp.3.weight", (1, 128))]:
        assert tuple(sd[key].shape) == shape, key
    assert sum(p.numel() for p in m.parameters()) == 951821
    lp = params.LatticeformerParams().parseFromArgs(params.ModelParams()).getLayerParameters(2)
    assert lp.scale_real == 1.4 and lp.layer_index == 2 and lp.cos_abs == 0 and lp.value_pe_angle_real == 64


def test_a_reference_checkpoint_loads_strictly():
    """The names and shapes below are what the reference's modules register for its default configuration
    (models/latticeformer.py:113,189; models/indexed_latticeformer_encoder.py:796-804;
    models/indexed_lattice_multi_head_attention_cuda.py:1042-1098), under the prefix its trainer's averaged model
    gives them (demo.py:75-79), next to entries a checkpoint also holds and the loader must ignore."""
    from crystalframer_amd import latticeformer
    gen = torch.Generator().manual_seed(5)
    shapes = {"input_embeddings.weight": (128, 98), "mlp.0.weight": (128, 128), "mlp.0.bias": (128,),
              "mlp.3.weight": (1, 128), "mlp.3.bias": (1,)}
    for li in range(4):
        pre = f"encoder.layers.{li}."
        shapes.update({pre + "linear1.weight": (512, 128), pre + "linear1.bias": (512,),
                       pre + "linear2.weight": (128, 512), pre + "linear2.bias": (128,)})
        at = pre + "self_attn."
        shapes.update({at + "gauss_scale": (2,), at + "atten_scale": (1,), at + "q_proj_weight": (128, 128),
                       at + "k_proj_weight": (128, 128), at + "v_proj_weight": (128, 128), at + "in_proj_bias": (384,),
                       at + "out_proj.weight": (128, 128), at + "out_proj.bias": (128,),
                       at + "lattice_pos_weights": (128,), at + "pe_dist_proj": (1, 8, 16, 64),
                       at + "proj_angle1": (1, 8, 16, 64), at + "proj_angle2": (1, 8, 16, 64),
                       at + "proj_angle3": (1, 8, 16, 64)})
    ckpt = {"swa_model.module." + k: torch.randn(v, generator=gen) for k, v in shapes.items()}
    ckpt.update({"model." + k: torch.zeros(v) for k, v in shapes.items()})
    ckpt["swa_model.n_averaged"] = torch.tensor(7)
    ckpt["target_std"], ckpt["target_mean"] = torch.tensor([2.5]), torch.tensor([-0.75])
    model = latticeformer.Latticeformer(params.ModelParams())
    assert set(model.state_dict()) == set(shapes)
    latticeformer.load_reference_checkpoint(model, ckpt)
    sd = model.state_dict()
    for k in shapes:
        if k.startswith("mlp.3"):
            continue
        assert torch.equal(sd[k], ckpt["swa_model.module." + k]), k
    assert torch.allclose(sd["mlp.3.weight"], ckpt["swa_model.module.mlp.3.weight"] * 2.5)
    assert torch.allclose(sd["mlp.3.bias"], ckpt["swa_model.module.mlp.3.bias"] * 2.5 - 0.75)
    # the three input projections are re-packed into one storage on first use without changing what was loaded
    at = model.encoder.layers[2].self_attn
    at._stacked_in_proj()
    assert torch.equal(at.k_proj_weight, ckpt["swa_model.module.encoder.layers.2.self_attn.k_proj_weight"])
    with pytest.raises(KeyError):
        latticeformer.load_reference_checkpoint(model, {"model.x": torch.zeros(1)})


def test_vectorised_frame_oracle_matches_loop_oracle():
    import helpers as Hh
    P = Hh.make_problem(num_crystals=5, atoms_hi=4, seed=71)
    f1, f2 = TO.frame_axes_max(P.q, P.k, P.a, P.rpos, P.tvecs, P.batch, P.edges, rvlen=P.rvlen, cutoff_radius=-3.5)
    g1, g2 = TO.frame_axes_max_vec(P.q, P.k, P.a, P.rpos, P.tvecs, P.batch, P.edges, rvlen=P.rvlen, cutoff_radius=-3.5)
    assert (f1 - g1).abs().max() < 1e-12 and (f2 - g2).abs().max() < 1e-12


def test_input_projection_weights_share_one_storage_without_changing_the_parameters():
    """The attention layer keeps q/k/v_proj_weight as adjacent row blocks of one matrix (the stacked
    projection then needs no concatenation).  Names, shapes and values stay the reference's; an
    optimizer step on the three parameters is seen through the stack; moving the module re-establishes it."""
    from crystalframer_amd import attention, params
    lat = params.LatticeformerParams()
    torch.manual_seed(3)
    m = attention.CrystalformerMultiheadAttentionCUDA(128, 8, params=lat)
    before = {k: v.clone() for k, v in m.state_dict().items()}
    st = m._stacked_in_proj()
    assert st.shape == (384, 128)
    assert m.q_proj_weight.data_ptr() == st.data_ptr()
    assert m.k_proj_weight.data_ptr() == st.data_ptr() + 128 * 128 * 4
    assert m.v_proj_weight.data_ptr() == st.data_ptr() + 2 * 128 * 128 * 4
    after = m.state_dict()
    assert list(after.keys()) == list(before.keys())
    for k in before:
        assert torch.equal(after[k], before[k]), k
    assert {n for n, _ in m.named_parameters()} >= {"q_proj_weight", "k_proj_weight", "v_proj_weight"}
    assert m._stacked_in_proj() is st                      # nothing to redo
    opt = torch.optim.SGD([m.q_proj_weight, m.k_proj_weight, m.v_proj_weight], lr=0.5)
    for p in (m.q_proj_weight, m.k_proj_weight, m.v_proj_weight):
        p.grad = torch.ones_like(p)
    opt.step()
    assert torch.equal(st[:128], before["q_proj_weight"] - 0.5)
    assert torch.equal(st[256:], before["v_proj_weight"] - 0.5)
    m2 = m.double()                                         # new storages per parameter
    st2 = m2._stacked_in_proj()
    assert st2.dtype == torch.float64 and st2 is not st
    assert torch.equal(st2[128:256], m2.k_proj_weight) and m2.k_proj_weight.data_ptr() == st2.data_ptr() + 128 * 128 * 8
    sd = {k: v.clone() for k, v in m2.state_dict().items()}
    m3 = attention.CrystalformerMultiheadAttentionCUDA(128, 8, params=lat).double()
    m3._stacked_in_proj()
    m3.load_state_dict(sd)                                  # copies into the shared storage
    assert torch.equal(m3._stacked_in_proj()[:128], sd["q_proj_weight"])


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits without touching a device."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 2
    assert "one GPU" in r.stderr
    assert r.stdout.strip() == ""
