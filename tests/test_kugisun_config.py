"""The Kugisun configuration on the CPU: what config.json gives, the order of the runs and whose
tensors each runs with, what is refused, the cache and state a layer asks for, the tensors a
model declares, a model folder written and read, and the plain implementation's own pieces by
hand."""
import copy
import json
import math
import os

import pytest
import torch

import kugisun_tiny as kt
import plain_kugisun as P
from zinfer_amd.config import (GatedDeltaRuleSpec, GatedExpertSpec, KugisunConfig, LayerNormSpec,
                               MaskedGqaAttentionSpec, MoeSpec, ParallelMixerSpec,
                               StreamBlockSpec, SwiGluSpec, entry_for)
from zinfer_amd.errors import ConfigError
from zinfer_amd.models.build import declare_tensors
from zinfer_amd.parts.base import KVNeed, StateNeed


def test_registry_finds_the_family_by_its_one_name():
    assert entry_for(kt.KG_A).config_type is KugisunConfig
    assert entry_for({"architecture": "Kugisun", "model_type": "qwen3"}).config_type is KugisunConfig


@pytest.mark.parametrize("name", sorted(kt.CONFIGS))
def test_sizes_and_constants_come_from_the_file(name):
    raw = kt.CONFIGS[name]
    cfg = kt.config_of(name)
    spec = cfg.model_spec()
    eps = raw["norm"]["eps"]
    assert (spec.vocab_size, spec.hidden_size, spec.max_positions) == \
        (raw["vocab"], raw["width"], raw["max_positions"])
    assert spec.tie_word_embeddings and spec.position_table_name == "pos"
    assert spec.streams == raw.get("streams")
    assert isinstance(spec.final_norm, LayerNormSpec) and spec.final_norm.eps == eps
    assert not spec.final_norm.centred and spec.final_norm.bias_name is None
    assert spec.final_norm.gain_offset == 1.0
    for number, block in zip(spec.layer_numbers, spec.layers):
        L = raw["layers"][number]
        assert "weights_of" not in L
        assert isinstance(block, StreamBlockSpec) and block.mixer_norm.eps == eps
        assert block.streams == raw.get("streams", 1) and block.learned == ("streams" in raw)
        assert block.mixer_norm.gain_offset == 1.0
        m = block.mixer
        assert isinstance(m, ParallelMixerSpec)
        assert (m.left_scale, m.right_scale) == (L["mixer"]["left_scale"], L["mixer"]["right_scale"])
        a, r = m.left, L["mixer"]["left"]
        assert isinstance(a, MaskedGqaAttentionSpec) and a.bias and a.qk_norm_per_head
        assert (a.n_heads, a.n_kv_heads, a.head_dim, a.value_dim, a.scale, a.qk_norm_eps) == \
            (r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["scale"], eps)
        assert a.window is None and a.chunk is None and a.softcap is None and not a.sink
        dims = r.get("rot", {}).get("dims", 0)
        if dims == 0:
            assert a.rotary is None
        else:
            assert a.rotary.interleaved and a.rotary.dims == dims and a.rotary.magnitude == 1.0
            base = r["rot"]["base"]
            assert a.rotary.frequencies == tuple(base ** (-2.0 * i / dims) for i in range(dims // 2))
        d, r = m.right, L["mixer"]["right"]
        assert isinstance(d, GatedDeltaRuleSpec)
        assert (d.n_heads, d.n_kv_heads, d.head_dim, d.value_dim, d.conv_taps, d.norm_eps,
                d.unit_eps, d.q_scale) == \
            (r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"], eps, 1e-6, None)
        f = block.feed_forward
        if L["mlp"] is None:
            assert f is None and block.ff_norm is None
        elif L["mlp"]["kind"] == "dense":
            assert isinstance(f, SwiGluSpec) and f.intermediate_size == L["mlp"]["ff"]
            assert (f.gate_name, f.up_name, f.down_name) == ("gate", "up", "down")
        else:
            q = L["mlp"]["router"]
            assert isinstance(f, MoeSpec) and f.scoring == "softmax_all" and not f.normalize
            assert f.group_mark == 1 and f.correction_name == "correction"
            assert (f.n_experts, f.n_identity, f.top_k, f.weight_scale) == \
                (q["experts"], q.get("identity", 0), q["top"], q.get("scale", 1.0))
            assert f.groups == (None if q["groups"] is None
                                else (q["groups"]["count"], q["groups"]["keep"]))
            assert isinstance(f.expert, GatedExpertSpec) and f.expert.limit is None
            assert f.expert.intermediate_size == L["mlp"]["expert"]["ff"]
            if L["mlp"]["shared"] is None:
                assert f.shared is None and f.shared_gate_name is None
            else:
                assert f.shared.intermediate_size == L["mlp"]["shared"]["ff"]
                assert f.shared_gate_name == "sg"
    assert cfg.to_dict() == raw and cfg.vocab_size == raw["vocab"]


def test_the_order_of_the_runs_and_whose_tensors_they_use():
    cfg = kt.config_of("A")
    assert cfg.layer_numbers == (0, 1, 2) and cfg.order == (0, 1, 2, 1, 1)
    spec = cfg.model_spec()
    assert [e.layer for e in spec.schedule] == [0, 1, 2, 1, 1]
    assert all(e.cache_of is None and not e.reentry for e in spec.schedule)
    d = kt.config_of("D")
    assert d.layer_numbers == (0, 1, 3) and d.order == (0, 1, 1, 2)
    # the oracle walks the same way
    assert [P.weights_layer(kt.KG_A, i) for i in range(5)] == [0, 1, 2, 1, 1]
    # a layer in the middle that brings no tensors: the ones behind it keep their numbers
    raw = copy.deepcopy(kt.KG_B)
    raw["layers"] = [raw["layers"][0], dict(raw["layers"][0], weights_of=0), raw["layers"][1]]
    c = KugisunConfig.from_dict(raw)
    assert c.layer_numbers == (0, 2) and c.order == (0, 0, 1)
    names = declare_tensors(c.model_spec())
    assert "l2.norm1" in names and not any(n.startswith("l1.") for n in names)


def test_what_the_configuration_refuses():
    def broken(change):
        raw = copy.deepcopy(kt.KG_A)
        change(raw)
        with pytest.raises(ConfigError):
            KugisunConfig.from_dict(raw).model_spec()

    broken(lambda r: r.pop("vocab"))
    broken(lambda r: r.pop("max_positions"))
    broken(lambda r: r.update(layers=[]))
    broken(lambda r: r["norm"].update(eps=-1.0))
    broken(lambda r: r["layers"][0].update(type="attention"))
    broken(lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=3))
    broken(lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=5))
    broken(lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=14))
    broken(lambda r: r["layers"][0]["mixer"]["right"].update(kv_heads=3))
    broken(lambda r: r["layers"][0]["mixer"]["right"].pop("conv"))
    broken(lambda r: r["layers"][0]["mixer"].pop("left_scale"))
    broken(lambda r: r["layers"][0]["mlp"].update(kind="sparse"))
    broken(lambda r: r["layers"][1]["mlp"]["router"].update(top=7))
    broken(lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(count=4))
    broken(lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(keep=4))
    broken(lambda r: r["layers"][3].update(weights_of=9))
    broken(lambda r: r["layers"][3].update(weights_of=4))        # 3 -> 4 -> 3
    broken(lambda r: r.update(streams=0))
    # what the kernels do not take is refused when the model is put together
    raw = copy.deepcopy(kt.KG_A)
    raw["layers"][0]["mixer"]["right"].update(dim=300)
    with pytest.raises(ConfigError):
        declare_tensors(KugisunConfig.from_dict(raw).model_spec())
    raw = copy.deepcopy(kt.KG_A)
    raw["streams"] = 9
    with pytest.raises(ConfigError):
        declare_tensors(KugisunConfig.from_dict(raw).model_spec())


def test_cache_needs_and_declared_tensors():
    import zinfer_amd.parts  # noqa: F401  (registers the parts)
    from zinfer_amd.models.decoder import DecoderModel
    from zinfer_amd.parts import BuildContext
    from zinfer_amd import ops
    spec = kt.config_of("A").model_spec()
    model = DecoderModel(spec, BuildContext(torch.float32, torch.device("meta")))
    needs = model.cache_needs()
    assert len(needs) == 5 and needs[1] == needs[3] == needs[4] and needs[0] != needs[1]
    for need, e in zip(needs, spec.schedule):
        block = spec.layers[e.layer]
        a, d = block.mixer.left, block.mixer.right
        kv = [n for n in need if isinstance(n, KVNeed)]
        st = [n for n in need if isinstance(n, StateNeed)]
        assert len(need) == 2 and len(kv) == 1 and len(st) == 1
        assert kv[0] == KVNeed(a.n_kv_heads, a.head_dim, None, value_dim=a.value_dim, chunk=None)
        # the matrices with the key size padded for the kernel, then taps - 1 rows of q, k and v
        r, lanes = ops.delta_plan(d.head_dim)
        assert r * lanes >= d.head_dim
        rows = (d.conv_taps - 1) * (2 * d.n_kv_heads * d.head_dim + d.n_heads * d.value_dim)
        assert st[0].dtype == torch.float32
        assert st[0].shape[0] >= d.n_heads * d.value_dim * r * lanes + rows
    names = declare_tensors(spec)
    for n in ("embed", "pos", "final.norm", "l0.norm1", "l0.norm2", "l0.hc1.in", "l0.hc1.mix",
              "l0.hc2.out", "l0.mix.left.q", "l0.mix.left.q.b", "l0.mix.left.k.norm",
              "l0.mix.left.o", "l0.mix.right.q.conv", "l0.mix.right.A_log", "l0.mix.right.dt_bias",
              "l0.mix.right.b", "l0.mix.right.a", "l0.mix.right.g", "l0.mix.right.norm",
              "l0.mlp.gate", "l1.mlp.router", "l1.mlp.correction", "l1.mlp.e4.down",
              "l1.mlp.shared.sg", "l1.mlp.shared.up", "l2.norm1", "l2.hc1.out"):
        assert n in names, n
    assert names["head"].optional
    for n in ("l2.norm2", "l2.hc2.in", "l2.mlp.gate", "l3.norm1", "l4.norm1", "l1.mlp.e5.gate"):
        assert n not in names, n
    assert names["l1.mlp.router"].shape == (6, 48) and names["l1.mlp.correction"].shape == (6,)
    assert names["l0.hc1.mix"].shape == (3, 3) and names["l0.mix.left.q.norm"].shape == (12,)
    assert names["l0.mix.right.v.conv"].shape == (40, 3) and names["pos"].shape == (512, 48)
    # no copies named: no coefficients
    plain = declare_tensors(kt.config_of("C").model_spec())
    assert not any(".hc" in n for n in plain)
    # every padded key size the kernel knows
    assert [ops.delta_plan(d) for d in (1, 8, 10, 12, 16, 24, 32, 40, 64, 96, 128, 256)] == \
        [(8, 1), (8, 1), (12, 1), (12, 1), (8, 2), (12, 2), (8, 4), (12, 4), (8, 8), (12, 8),
         (8, 16), (16, 16)]


def test_a_folder_written_and_read(tmp_path):
    from zinfer_amd.config import load_config
    from zinfer_amd.weights.loader import load_tensors
    from zinfer_amd.weights.safetensors_io import write_safetensors
    path = str(tmp_path)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(kt.KG_B, f)
    w = kt.weights_of("B", dtype=torch.bfloat16)
    write_safetensors(os.path.join(path, "model.safetensors"), w)
    cfg = load_config(path)
    assert isinstance(cfg, KugisunConfig)
    got = load_tensors(path, declare_tensors(cfg.model_spec()))
    assert set(got) == set(w) and "head" not in got
    assert all(torch.equal(got[n], w[n]) for n in w)


def test_the_plain_pieces_by_hand():
    # the norm's weight lies around zero
    v = torch.tensor([[3.0, -4.0]])
    assert torch.allclose(P.norm_one_plus(v, torch.tensor([0.0, 1.0]), 0.0),
                          torch.tensor([[3.0, -8.0]], dtype=P.F64) / math.sqrt(12.5))
    # neighbours turn together, elements beyond ``dims`` pass
    x = torch.tensor([[[1.0, 0.0, 0.0, 2.0, 5.0, 6.0]]])
    y = P.rotate_pairs(x, torch.tensor([1]), 4, 4.0)
    a0, a1 = 1.0, 4.0 ** -0.5
    want = [math.cos(a0), math.sin(a0), -2 * math.sin(a1), 2 * math.cos(a1), 5.0, 6.0]
    assert torch.allclose(y[0, 0], torch.tensor(want, dtype=P.F64))
    # the last tap is the token's own; zeros before the start
    c = P.short_convolution(torch.tensor([[1.0], [2.0], [3.0]]), torch.tensor([[10.0, 1.0]]))
    assert c[:, 0].tolist() == [1.0, 12.0, 23.0]
    # one token of the delta rule from a zero matrix: S = beta k v^T, o = beta (q . k) v
    q, k, val = torch.tensor([[1.0, 2.0]]), torch.tensor([[0.5, 0.0]]), torch.tensor([[3.0, 4.0, 5.0]])
    o, S = P.delta_rule(q.double(), k.double(), val.double(), torch.tensor([0.5]).double(),
                        torch.tensor([0.9]).double())
    assert torch.allclose(o[0], 0.5 * 0.5 * val[0].double())
    assert torch.allclose(S, 0.5 * torch.outer(k[0], val[0]).double())
    # a second token with the same key takes the matrix towards its own value
    o2, S2 = P.delta_rule(torch.cat([q, q]).double(), torch.tensor([[1.0, 0.0]] * 2).double(),
                          torch.tensor([[1.0], [5.0]]).double(), torch.tensor([1.0, 1.0]).double(),
                          torch.tensor([1.0, 1.0]).double())
    assert S2[0, 0] == 5.0 and o2[:, 0].tolist() == [1.0, 5.0]
    # the router: a correction changes the choice and not the weights; a group is shut out
    # although it holds the best output; negative choice scores still choose
    h = torch.eye(4, dtype=P.F64)[:1]
    R = torch.tensor([[2.0, 0, 0, 0], [1.0, 0, 0, 0], [3.0, 0, 0, 0], [-4.0, 0, 0, 0]])
    s = torch.softmax(R[:, 0].double(), dim=0)
    r = {"top": 2, "scale": 2.0, "groups": None}
    ids, wts = P.route(h, R, torch.zeros(4), r)
    assert ids[0].tolist() == [2, 0] and torch.allclose(wts[0], 2.0 * s[[2, 0]])
    ids, wts = P.route(h, R, torch.tensor([0.0, 1.0, 0.0, 0.0]), r)
    assert ids[0].tolist() == [1, 2] and torch.allclose(wts[0], 2.0 * s[[1, 2]])
    r = {"top": 2, "groups": {"count": 2, "keep": 1}}
    ids, wts = P.route(h, R, torch.tensor([0.0, 0.0, -5.0, 0.5]), r)
    # marks: group 0 = max(s0, s1), group 1 = max(s2 - 5, s3 + 0.5): group 1 wins with 0.5+
    assert sorted(ids[0].tolist()) == [2, 3] and ids[0].tolist() == [3, 2]
    assert torch.allclose(wts[0], s[[3, 2]])
    # an output without an expert hands the input on
    f = {"kind": "moe", "router": {"experts": 1, "identity": 1, "top": 1, "groups": None},
         "expert": {"ff": 2}, "shared": None}
    w = {"router": torch.tensor([[0.0, 0.0], [5.0, 0.0]]), "correction": torch.zeros(2),
         "e0.gate": torch.ones(2, 2), "e0.up": torch.ones(2, 2), "e0.down": torch.ones(2, 2)}
    x = torch.tensor([[1.0, 3.0]], dtype=P.F64)
    share = torch.softmax(torch.tensor([0.0, 5.0], dtype=P.F64), dim=0)[1]
    assert torch.allclose(P.mixture(x, w, f), share * x)
    # one copy without coefficients is the plain sum
    X = P.stream_step([torch.ones(1, 2, dtype=P.F64)], {}, 1, lambda u: 2 * u)
    assert X[0].tolist() == [[3.0, 3.0]]
    # all copies at once from the old ones
    w = {"hc1.in": torch.tensor([1.0, 0.0]), "hc1.mix": torch.tensor([[0.0, 1.0], [1.0, 0.0]]),
         "hc1.out": torch.tensor([1.0, -1.0])}
    X = P.stream_step([torch.tensor([[1.0]], dtype=P.F64), torch.tensor([[10.0]], dtype=P.F64)],
                      w, 1, lambda u: 100 * u)
    assert [x.item() for x in X] == [110.0, -99.0]
