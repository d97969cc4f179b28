"""Roravik on the CPU: configuration reading and refusals, run order, tensor names, the parts a layer is made of,
the inner width of the decay taken from the checkpoint's shapes, and the cache's bookkeeping for the states."""
import copy
import json

import pytest
import torch

from rocml_amd.cache import Cache
from rocml_amd.config import architecture_of
from rocml_amd.engine.model import DecoderModel
from rocml_amd.errors import ConfigError
from rocml_amd.parts.base import CompositeRequest, KVCacheRequest, StateRequest
from tests import roravik_models as rm
from tests.plain import roravik_plain as plain


def _spec(cfg):
    arch = architecture_of(cfg)
    return arch, arch.to_spec(arch.read_config(cfg))


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_tensor_names_and_shapes(name):
    cfg, _ = rm.CONFIGS[name]
    arch, spec = _spec(cfg)
    model = DecoderModel(spec, torch.float32, device="meta")
    names = arch.checkpoint_names(spec)
    mine = {names[k]: tuple(p.shape) for k, p in model.param_specs().items()}
    unused = set(arch.unused_tensors(spec))
    theirs = rm.tensor_shapes(cfg)
    assert mine == {k: v for k, v in theirs.items() if k not in unused}
    assert unused == {f"l{i}.norm2{b}" for i, l in enumerate(cfg["layers"]) if l.get("mlp") is None for b in ("", "b")}
    assert "head" not in mine, "the logits come from the embedding's table"
    assert model.kernel_families()[:3] == ("elementwise", "gemm", "attention")
    assert "recurrent" in model.kernel_families() and "moe" in model.kernel_families()


def test_run_order_follows_the_loop():
    for name in ["A", "B", "C", "D"]:
        cfg, _ = rm.CONFIGS[name]
        _, spec = _spec(cfg)
        mine = [(e.layer, e.add_embedding) for e in spec.schedule]
        assert mine == plain.layer_order(cfg), name
        assert all(e.reads_cache_of is None and e.offset_row is None for e in spec.schedule)
    _, spec = _spec(rm.CFG_A)
    assert [(e.layer, e.add_embedding) for e in spec.schedule] == \
        [(0, False), (1, False), (2, False), (1, True), (2, False), (3, False), (4, False)]
    model = DecoderModel(spec, torch.float32, device="meta")
    assert len(model.cache_requests()) == 7, "every pass has a cache line of its own"


def test_spec_carries_every_constant():
    _, spec = _spec(rm.CFG_A)
    assert spec.tie_lm_head and spec.logit_softcap == 12.0 and spec.embed_scale == 8.5 and spec.head_spec().softcap == 12.0
    assert spec.final_norm.unit_offset and spec.final_norm.eps == 3e-6
    first, second, third, fourth, fifth = spec.layers
    for b in spec.layers:
        assert b.arrangement == "sandwich_norm"
        for norm in (b.mixer_norm, b.mixer_out_norm) + ((b.ffn_norm, b.ffn_out_norm) if b.ffn is not None else ()):
            assert norm.kind == "rmsnorm" and norm.unit_offset and norm.size == 72
    assert third.ffn is None and third.ffn_norm is None and third.ffn_out_norm is None
    assert not first.mixer.normed and first.mixer.branch_weights == (0.6, 0.9)
    (lname, left), (rname, right) = first.mixer.branches
    assert (lname, rname) == ("left", "right")
    assert (left.n_heads, left.n_kv_heads, left.head_dim, left.v_head_dim, left.scale, left.window) == (4, 2, 24, 16, 0.9, 7)
    assert left.sink and left.sink_learned and left.softcap == 8.0 and left.conv == 3 and left.qk_norm is None and not left.bias
    assert (left.position.rot_dim, left.position.theta) == (12, 5000.0)
    assert (right.n_heads, right.head_dim, right.decay_rank, right.eps) == (3, 17, 5, 3e-6)
    ret = second.mixer
    assert ret.kind == "retention" and (ret.n_heads, ret.head_dim, ret.v_head_dim, ret.decay) == (2, 20, 36, (0.9, 0.995))
    assert (ret.position.rot_dim, ret.position.theta) == (20, 10000.0)
    assert (second.ffn.activation, second.ffn.limit, second.ffn.up_offset, second.ffn.intermediate) == ("sigmoid_1702", 1.5, 1.0, 88)
    moe = first.ffn
    assert (moe.n_experts, moe.top, moe.intermediate, moe.groups, moe.weighting, moe.correction, moe.group_score) == \
        (6, 2, 24, (2, 1), "sigmoid", True, "top2_sum")
    assert moe.shared_intermediate == 40 and moe.shared_gate and moe.sum_eps == 1e-20
    assert fourth.ffn.shared_intermediate is None and not fourth.ffn.shared_gate and fourth.ffn.groups == (3, 2)
    assert fifth.ffn.groups is None and fifth.ffn.top == 1


def test_refusals():
    def broken(change):
        cfg = copy.deepcopy(rm.CFG_A)
        change(cfg)
        with pytest.raises(ConfigError):
            _spec(cfg)
    broken(lambda c: c["layers"][0].update(type="attention"))
    broken(lambda c: c["layers"][1]["mixer"].update(decay=[0.9]))
    broken(lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3))
    broken(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=13))
    broken(lambda c: c["layers"][0]["mixer"].pop("left_scale"))
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=7))
    broken(lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4))
    broken(lambda c: c["loop"].update(stop=9))
    broken(lambda c: c["loop"].update(start=3))
    broken(lambda c: c.pop("logit_softcap"))
    broken(lambda c: c["layers"][1]["mlp"].pop("limit"))
    cfg = copy.deepcopy(rm.CFG_A)
    cfg["architecture"] = "Roravic"
    with pytest.raises(Exception):
        architecture_of(cfg)
    # a configuration survives the round trip through its typed form
    arch = architecture_of(rm.CFG_A)
    assert arch.read_config(arch.read_config(rm.CFG_A).to_dict()) == arch.read_config(rm.CFG_A)


def test_decay_rank_comes_from_the_shapes(tmp_path):
    cfg, seed = rm.CONFIGS["A"]
    arch = architecture_of(cfg)
    bare = json.loads(json.dumps(cfg))
    for lay in bare["layers"]:
        if lay["type"] == "parallel":
            lay["mixer"]["right"].pop("decay_rank")
    typed = arch.read_config(bare)
    shapes = rm.tensor_shapes(cfg)
    spec = arch.to_spec(arch.refine_config(typed, shapes))
    assert [b.mixer.branches[1][1].decay_rank for b in spec.layers if b.mixer.kind == "parallel"] == [5, 8, 3]
    # and the loader does so by itself
    from rocml_amd.weights import load_model
    path = rm.write_model(str(tmp_path / "m"), cfg, rm.random_tensors(cfg, seed))
    assert "decay_rank" not in open(f"{path}/config.json").read()
    model = load_model(path, dtype="float32", device="cpu")
    assert model.blocks[0].mixer.children["right"].spec.decay_rank == 5


def test_cache_lines_and_states():
    _, spec = _spec(rm.CFG_A)
    model = DecoderModel(spec, torch.float32, device="meta")
    requests = model.cache_requests()
    assert isinstance(requests[0], CompositeRequest)
    left, right = requests[0].parts
    assert left.parts == (KVCacheRequest(2, 24, 7, v_head_dim=16, chunk=None), StateRequest((2, 4 * 24 + 2 * 24 + 2 * 16)))
    assert right.parts == (StateRequest((3, 17, 17)), StateRequest((72,)))
    assert requests[1] == StateRequest((2, 36, 20)) and requests[3] == requests[1]
    cache = Cache(requests, max_tokens=256, dtype=torch.float32, device="cpu", max_seqs=3)
    g_conv, line_conv = cache.line(0, 0, 1)
    g_s, line_s = cache.line(0, 1, 0)
    g_prev, line_prev = cache.line(0, 1, 1)
    g_r1, line_r1 = cache.line(1)
    g_r3, line_r3 = cache.line(3)
    assert cache.line(0, 0, 0)[0].paged and not g_conv.paged and not g_s.paged
    assert (g_r1 is not g_r3) or line_r1 != line_r3, "the two passes of a layer keep their states apart"
    a = cache.new_sequence()
    cache.reserve([a], [70])
    cache.commit([a], [70])
    for g, line in ((g_conv, line_conv), (g_s, line_s), (g_prev, line_prev), (g_r1, line_r1), (g_r3, line_r3)):
        g.state[line, a].fill_(3.0)
    cache.free_sequence(a)
    b = cache.new_sequence()
    assert b == a
    for g, line in ((g_conv, line_conv), (g_s, line_s), (g_prev, line_prev), (g_r1, line_r1), (g_r3, line_r3)):
        assert float(g.state[line, b].abs().max()) == 0.0, "a slot that is used again starts from zero states"
    cache.free_sequence(b)
    cache.check()


def test_choice_of_experts_in_the_plain_implementation():
    """The oracle's own choice, on a case made by hand: the correction moves the choice, not the weights, and a
    group wins by the sum of its two best."""
    z = torch.tensor([[2.0, -9.0, -9.0, 1.5, 1.4, -9.0]], dtype=torch.float64)
    none = torch.zeros(6, dtype=torch.float64)
    chosen, w = plain.choose_experts(z, none, {"top": 2, "groups": {"count": 2, "keep": 1}})
    # group 0 holds the best expert, but group 1's two best add up to more
    assert chosen.tolist() == [[3, 4]]
    s = torch.sigmoid(z[0, [3, 4]])
    assert torch.allclose(w[0], s / s.sum())
    corr = torch.tensor([0.0, 5.0, 0.0, 0.0, 0.0, 0.0], dtype=torch.float64)
    chosen, w = plain.choose_experts(z, corr, {"top": 2, "groups": {"count": 2, "keep": 1}})
    assert chosen.tolist() == [[1, 0]] and float(w[0, 0]) < 1e-3, "expert 1 is chosen for its correction and weighs by its score"
    chosen, _ = plain.choose_experts(z, none, {"top": 2, "groups": None})
    assert chosen.tolist() == [[0, 3]]


def test_random_model_folder_has_the_checkpoint_names(tmp_path):
    from safetensors import safe_open
    from rocml_amd.config.catalog import resolve
    from rocml_amd.weights import write_model_dir
    cfg = resolve("roravik-tiny").entry.config
    path = write_model_dir(str(tmp_path / "m"), cfg, 5, dtype=torch.bfloat16, norm_jitter=True)
    arch, spec = _spec(cfg)
    model = DecoderModel(spec, torch.float32, device="meta")
    names = arch.checkpoint_names(spec)
    with safe_open(f"{path}/model.safetensors", "pt") as f:
        found = {k: tuple(f.get_slice(k).get_shape()) for k in f.keys()}
    assert found == {names[k]: tuple(p.shape) for k, p in model.param_specs().items()}
    assert architecture_of(json.load(open(f"{path}/config.json"))).name == "Roravik"
