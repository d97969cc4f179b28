"""Sogavik on the CPU: configuration reading, tensor names, the parts a layer is made of, the stretched
rotation's frequencies, and the cache's bookkeeping for the matrix memory's state."""
import copy
import json

import pytest
import torch

from rocml_amd.cache import Cache
from rocml_amd.config import architecture_of
from rocml_amd.engine.model import DecoderModel
from rocml_amd.errors import ConfigError
from rocml_amd.parts.base import BuildContext, CompositeRequest, KVCacheRequest, StateRequest
from tests import sogavik_models as sm
from tests.plain import sogavik_plain as plain


def _spec(cfg):
    arch = architecture_of(cfg)
    return arch, arch.to_spec(arch.read_config(cfg))


@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_tensor_names_and_shapes(name):
    cfg, _ = sm.CONFIGS[name]
    arch, spec = _spec(cfg)
    model = DecoderModel(spec, torch.float32, device="meta")
    names = arch.checkpoint_names(spec)
    mine = {names[k]: tuple(p.shape) for k, p in model.param_specs().items()}
    unused = set(arch.unused_tensors(spec))
    theirs = sm.tensor_shapes(cfg)
    assert mine == {k: v for k, v in theirs.items() if k not in unused}
    # the second norm of a layer without a feed-forward is in the file and not read
    assert unused == {f"l{i}.norm2{b}" for i, l in enumerate(cfg["layers"]) if l.get("mlp") is None for b in ("", ".b")}
    assert model.kernel_families()[:3] == ("elementwise", "gemm", "attention")
    assert "recurrent" in model.kernel_families() and "moe" in model.kernel_families()


def test_spec_carries_every_constant():
    cfg, _ = sm.CONFIGS["A"]
    _, spec = _spec(cfg)
    assert spec.final_norm.kind == "layernorm" and spec.final_norm.eps == 3e-6 and not spec.tie_lm_head
    assert [t.name for t in spec.tables] == ["token_side"] and (spec.tables[0].rows, spec.tables[0].cols) == (211, 4 * 5)
    first, second, third, fourth = spec.layers
    assert all(b.arrangement == "sublayer_norm" and b.mixer_norm.kind == "layernorm" for b in spec.layers)
    att = first.mixer
    assert (att.n_heads, att.n_kv_heads, att.head_dim, att.v_head_dim, att.scale, att.window) == (4, 2, 24, 16, 0.9, 7)
    assert att.bias and att.o_bias is False and att.gate and att.gate_per_head and att.qk_norm_span == "projection"
    assert att.qk_norm.size == 4 * 24 and (att.position.rot_dim, att.position.theta) == (12, 5000.0)
    st = att.position.stretch
    assert (st.factor, st.original, st.fast, st.slow) == (3.0, 64.0, 8.0, 2.0)
    assert (first.ffn.n_experts, first.ffn.top, first.ffn.intermediate, first.ffn.weighting, first.ffn.router_bias) == \
        (6, 2, 24, "softmax_chosen", True)
    assert [b.side.column0 for b in spec.layers] == [0, 5, 10, 15] and first.side.dim == 5 and first.side_norm.kind == "rmsnorm"
    (lname, left), (rname, right) = second.mixer.branches
    assert (lname, rname) == ("left", "right") and second.mixer.weight == 0.5
    assert not left.gate and left.position.stretch is None and left.position.rot_dim == 16 and left.window == 33
    assert (right.n_heads, right.head_dim, right.v_head_dim, right.gate_cap, right.floor) == (2, 20, 36, 8.0, 1e-6)
    assert second.ffn is None and second.ffn_norm is None
    assert third.ffn.top == 1 and fourth.ffn.top == fourth.ffn.n_experts == 3
    # a model without side input has no table and no side sublayer
    _, plain_spec = _spec(sm.CONFIGS["D"][0])
    assert plain_spec.tables == () and all(b.side is None for b in plain_spec.layers)
    # a layer without a window or a rotation
    _, c = _spec(sm.CONFIGS["C"][0])
    assert c.layers[1].mixer.branches[0][1].window is None and c.layers[1].mixer.branches[0][1].position is None


def test_config_round_trip_and_refusals():
    cfg, _ = sm.CONFIGS["B"]
    arch = architecture_of(cfg)
    assert arch.read_config(arch.read_config(cfg).to_dict()) == arch.read_config(cfg)
    for path, value in ([("layers", 0, "type"), "serial"], [("layers", 1, "mixer", "kv_heads"), 3],
                        [("layers", 0, "mixer", "right", "gate_cap"), 0], [("layers", 1, "mlp", "router", "top"), 17],
                        [("layers", 1, "mixer", "rot", "dims"), 7], [("layers", 1, "mixer", "rot", "dims"), 130],
                        [("layers", 1, "mixer", "rot", "scaling", "factor"), -1.0], [("layers", 1, "mixer", "mask", "size"), 0],
                        [("norm", "eps"), -1.0], [("token_side", "dim"), 0], [("layers", 0, "mlp", "kind"), "dense"],
                        [("width",), 0]):
        bad = copy.deepcopy(cfg)
        at = bad
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(ConfigError):
            arch.read_config(bad)


@pytest.mark.parametrize("rot", [{"base": 200000.0, "dims": 64, "scaling": {"factor": 5.0, "original": 128, "fast": 16.0, "slow": 1.0}},
                                 {"base": 5000.0, "dims": 12, "scaling": {"factor": 3.0, "original": 64, "fast": 8.0, "slow": 2.0}},
                                 {"base": 100.0, "dims": 20, "scaling": {"factor": 1.0, "original": 16, "fast": 2.0, "slow": 1.0}},
                                 {"base": 10000.0, "dims": 2, "scaling": {"factor": 16.0, "original": 4096, "fast": 24.0, "slow": 1.5}},
                                 {"base": 300.0, "dims": 4}])
def test_stretched_frequencies(rot):
    """The rotation part's frequencies and magnitude against the plain function; with a stretch, some frequencies
    must stay, some be divided by the factor and (where the ramp is long enough) some lie between."""
    from rocml_amd.config.spec import RopeSpec, RopeStretch
    from rocml_amd.parts.rope import RopeNeox
    sc = rot.get("scaling")
    stretch = None if sc is None else RopeStretch(sc["factor"], sc["original"], sc["fast"], sc["slow"])
    part = RopeNeox(RopeSpec(head_dim=rot["dims"] + 8, rot_dim=rot["dims"], theta=rot["base"], stretch=stretch),
                    BuildContext(dtype=torch.float32, device=torch.device("cpu")))
    f, mag = plain.rotary_frequencies(rot)
    assert torch.allclose(part.inv_freq, torch.tensor(f, dtype=torch.float64), rtol=1e-14, atol=0)
    assert abs(part.magnitude - mag) < 1e-15
    if rot["dims"] == 64:
        bare = [rot["base"] ** (-2.0 * i / 64) for i in range(32)]
        ratio = [a / b for a, b in zip(f, bare)]
        assert ratio[0] == 1.0 and abs(ratio[-1] - 0.2) < 1e-12 and any(0.21 < r < 0.99 for r in ratio)


def test_cache_lines_of_the_matrix_memory():
    from rocml_amd import ops
    cfg, _ = sm.CONFIGS["A"]
    _, spec = _spec(cfg)
    model = DecoderModel(spec, torch.float32, device="meta")
    requests = model.cache_requests()
    assert requests[0] == KVCacheRequest(2, 24, 7, v_head_dim=16, chunk=None)
    assert isinstance(requests[1], CompositeRequest)
    kv, inner = requests[1].parts
    assert kv == KVCacheRequest(3, 16, 33, v_head_dim=40, chunk=None)
    tiles = ops.mlstm_tiles(36)
    assert tiles == 2
    assert inner.parts == (StateRequest((2, 36, 20)), StateRequest((2, tiles, 20)), StateRequest((2, tiles)))
    cache = Cache(requests, max_tokens=256, dtype=torch.float32, device="cpu", max_seqs=3)
    g_s, line_s = cache.line(1, 1, 0)
    g_n, _ = cache.line(1, 1, 1)
    g_m, line_m = cache.line(1, 1, 2)
    assert not g_s.paged and g_s is not g_n and g_n is not g_m and cache.line(1, 0)[0].paged
    a = cache.new_sequence()
    cache.reserve([a], [70])
    cache.commit([a], [70])
    g_s.state[line_s, a].fill_(3.0)
    g_m.state[line_m, a].fill_(-2.0)
    cache.free_sequence(a)
    b = cache.new_sequence()
    assert b == a and float(g_s.state[line_s, b].abs().max()) == 0.0 and float(g_m.state[line_m, b].abs().max()) == 0.0, \
        "a slot that is used again starts from a zero state and a running maximum of zero"
    cache.free_sequence(b)
    cache.check()


def test_random_model_folder_has_the_checkpoint_names(tmp_path):
    """``init`` for a catalog entry of this design writes config.json and every tensor under its checkpoint name."""
    from safetensors import safe_open
    from rocml_amd.config.catalog import resolve
    from rocml_amd.weights import write_model_dir
    cfg = resolve("sogavik-tiny").entry.config
    path = write_model_dir(str(tmp_path / "m"), cfg, 5, dtype=torch.bfloat16, norm_jitter=True)
    arch, spec = _spec(cfg)
    model = DecoderModel(spec, torch.float32, device="meta")
    names = arch.checkpoint_names(spec)
    with safe_open(f"{path}/model.safetensors", "pt") as f:
        found = {k: tuple(f.get_slice(k).get_shape()) for k in f.keys()}
    assert found == {names[k]: tuple(p.shape) for k, p in model.param_specs().items()}
    assert "side.embed" in found and found["side.embed"] == (cfg["vocab"], len(cfg["layers"]) * cfg["token_side"]["dim"])
    assert architecture_of(json.load(open(f"{path}/config.json"))).name == "Sogavik"
