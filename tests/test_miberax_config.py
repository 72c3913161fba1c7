"""Miberax without a GPU: the configuration's reader, the list of parts it becomes, tensor names and
shapes against the plain implementation's own table, the cache store's composite caches, and the
plain implementation's mechanisms against each other."""

from __future__ import annotations

import copy

import pytest
import torch

import plain_miberax as P


def cfg_dict():
    left = lambda chunk, rot: {"heads": 6, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.2,
                               **({"mask": {"size": chunk}} if chunk else {}),
                               **({"rot": {"dims": rot, "base": 5000.0, "scaling": {"factor": 4.0}}} if rot else {})}
    right = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "conv": 3}
    moe = {"kind": "moe", "expert": {"ff": 20, "limit": 0.9},
           "router": {"experts": 7, "top": 2, "identity": 1, "scale": 1.5, "groups": {"count": 4, "keep": 3}},
           "shared": {"ff": 28, "limit": 1.1}}
    return {"architecture": "Miberax", "vocab": 50, "width": 48, "norm": {"eps": 1e-5, "groups": 3},
            "layers": [{"type": "parallel", "mixer": {"left": left(9, 8), "right": right}, "mlp": {"kind": "dense", "ff": 80}},
                       {"type": "parallel", "mixer": {"left": left(0, 0), "right": right}, "mlp": None},
                       {"type": "parallel", "mixer": {"left": left(100, 16), "right": right}, "mlp": moe}]}


def build(raw):
    from dli_amd.config.registry import resolve_architecture
    from dli_amd.parts import Runtime
    from dli_amd.parts.model import Model
    import dli_amd.architectures  # noqa: F401

    arch = resolve_architecture(raw)
    cfg = arch.parse_config(raw)
    return cfg, Model(arch.build_spec(cfg), Runtime(torch.device("cpu"), torch.float32))


def test_config_is_read_and_becomes_parts():
    from dli_amd.parts import CompositeCacheSpec, PagedKVSpec, StateSpec

    cfg, model = build(cfg_dict())
    assert cfg.architecture == "Miberax" and (cfg.vocab, cfg.width, cfg.norm_eps, cfg.norm_groups) == (50, 48, 1e-5, 3)
    assert [(l.left.chunk, l.left.rot_dims, l.left.rot_factor) for l in cfg.layers] == [(9, 8, 4.0), (0, 0, 1.0), (100, 16, 4.0)]
    assert [None if l.mlp is None else l.mlp.kind for l in cfg.layers] == ["dense", None, "moe"]
    m = cfg.layers[2].mlp
    assert (m.experts, m.top, m.identity, m.scale, m.groups, m.groups_kept, m.ff, m.limit, m.shared_ff, m.shared_limit) == \
        (7, 2, 1, 1.5, 4, 3, 20, 0.9, 28, 1.1)
    mixers = [l.parts["mixer"] for l in model.layers]
    assert all(x.kind == "parallel_mixers" and list(x.branches) == ["left", "right"] for x in mixers)
    lefts = [x.branches["left"] for x in mixers]
    assert all(a.kind == "scored_attention" and not a.qk_unit and not a.sink and not a.output_gate for a in lefts)
    assert [a.chunk for a in lefts] == [9, 0, 100]
    tables = [a.position.rotary_table() for a in lefts]
    assert tables[1] is None and tables[0].pairing == "interleaved" and (tables[0].dim, tables[2].dim) == (8, 16)
    want = torch.pow(torch.tensor(5000.0, dtype=torch.float64), -2.0 * torch.arange(4, dtype=torch.float64) / 8) / 4.0
    assert (tables[0].inv_freq.double() - want).abs().max() < 1e-8
    assert [type(l.parts.get("feed_forward")).__name__ for l in model.layers] == ["PolyNormMLP", "NoneType", "RoutedExperts"]
    assert all(l.parts["mixer_norm"].kind == "group_rms_norm" and l.parts["mixer_norm"].groups == 3 for l in model.layers)
    specs = model.cache_specs()
    state = StateSpec((4 * 12 * 8 + 2 * (2 * 2 * 8 + 4 * 12),), torch.float32)
    assert specs[0] == specs[1] == specs[2] == CompositeCacheSpec((("left", PagedKVSpec(2, 16, 0, 24)), ("right", state)))
    assert model.head.tied and model.embedding.float32_rows


def test_tensor_names_and_shapes_are_the_plain_table():
    raw = cfg_dict()
    _, model = build(raw)
    table = P.tensor_shapes(raw)
    specs = model.weight_specs()
    assert set(specs) == set(table)
    for name, shape in table.items():
        assert specs[name].fits(tuple(shape)), (name, shape, specs[name].shape)


def test_what_is_not_implemented_is_refused():
    from dli_amd.config.errors import ConfigError

    def broken(change):
        raw = copy.deepcopy(cfg_dict())
        change(raw)
        with pytest.raises(ConfigError):
            build(raw)

    broken(lambda r: r["layers"][0].__setitem__("type", "serial"))
    broken(lambda r: r["layers"][0]["mixer"]["left"]["mask"].__setitem__("stride", 2))
    broken(lambda r: r["layers"][0]["mixer"]["left"]["rot"].__setitem__("dims", 7))
    broken(lambda r: r["layers"][0]["mixer"]["left"]["rot"]["scaling"].__setitem__("kind", "ntk"))
    broken(lambda r: r["layers"][0]["mixer"]["left"].__setitem__("kv_heads", 4))
    broken(lambda r: r["layers"][0]["mixer"]["right"].__setitem__("conv", 40))
    broken(lambda r: r["layers"][2]["mlp"].__setitem__("kind", "sparse"))
    broken(lambda r: r["layers"][2]["mlp"]["router"]["groups"].__setitem__("count", 3))   # 8 outputs in 3 groups
    broken(lambda r: r["layers"][2]["mlp"]["router"].__setitem__("top", 7))               # more than the kept groups hold
    broken(lambda r: r["norm"].__setitem__("groups", 5))
    broken(lambda r: r.pop("width"))


def test_composite_caches_in_the_store():
    from dli_amd.cache.store import CacheStore, flatten_specs, plan_groups
    from dli_amd.parts import CompositeCacheSpec, PagedKVSpec, Runtime, StateSpec

    a, b = PagedKVSpec(2, 16, 0, 24), PagedKVSpec(1, 8)
    st = StateSpec((10,), torch.float32)
    specs = [CompositeCacheSpec((("left", a), ("right", st))), None, b, CompositeCacheSpec((("x", st), ("y", b), ("z", a)))]
    assert flatten_specs(specs) == [a, st, None, b, st, b, a]
    groups, of = plan_groups(specs)
    assert groups == [a, b] and of == [0, -1, -1, 1, -1, 1, 0]
    store = CacheStore(Runtime(torch.device("cpu"), torch.float32), specs, num_pages=5, page_size=4, max_seqs=3)
    first, _, plain, last = store.layers
    assert first.kind == "composite" and set(first.members) == {"left", "right"} and plain.kind == "paged" and plain.group == 1
    assert first.members["left"].k_pages.shape == (5, 2, 4, 16) and first.members["left"].v_pages.shape == (5, 2, 24, 4)
    assert first.members["right"].state.shape == (4, 10) and last.members["x"].state.shape == (4, 10)
    # the two layers of each group have pages of their own
    assert first.members["left"].k_pages.data_ptr() != last.members["z"].k_pages.data_ptr()
    assert plain.k_pages.data_ptr() != last.members["y"].k_pages.data_ptr()
    assert first.members["right"].state.data_ptr() != last.members["x"].state.data_ptr()
    assert store.stateful and store.layers_per_group == [2, 2]
    reader = last.reader()
    assert not reader.writable and not any(c.writable for c in reader.members.values())


def test_plain_mechanisms_agree_with_their_definitions():
    torch.manual_seed(0)
    F = torch.float64
    # o is made from the state that already holds the token: one token, zero state
    q, k, v = torch.randn(1, 1, 4, dtype=F), torch.randn(1, 1, 4, dtype=F), torch.randn(1, 1, 3, dtype=F)
    o = P.gated_delta_rule(q, k, v, torch.tensor([[0.5]], dtype=F), torch.tensor([[0.9]], dtype=F))
    assert torch.allclose(o[0, 0], 0.5 * v[0, 0] * (k[0, 0] @ q[0, 0]))
    # a chunk of one position: every query sees itself alone
    vv = torch.randn(5, 1, 2, dtype=F)
    assert torch.allclose(P.chunked_attention(torch.randn(5, 2, 4, dtype=F), torch.randn(5, 1, 4, dtype=F), vv, 1.0, 1), vv.expand(5, 2, 2))
    # rotation keeps lengths and the products of a pair rotated alike depend on the distance alone
    x = torch.randn(1, 1, 8, dtype=F)
    a = P.rotate_interleaved(x.expand(2, 1, 8), torch.tensor([3, 10]), 6, 100.0, 2.0)
    b = P.rotate_interleaved(x.expand(2, 1, 8), torch.tensor([13, 20]), 6, 100.0, 2.0)
    assert torch.allclose(a.norm(dim=-1), x.norm(dim=-1).expand(2, 1)) and torch.equal(a[..., 6:], x.expand(2, 1, 8)[..., 6:])
    assert torch.allclose(a[0, 0] @ a[1, 0], b[0, 0] @ b[1, 0])
    # groups whose best choice score is not among the kept ones never win, also with negative scores
    t = {"r.router": torch.eye(6, dtype=F) * 0.0, "r.correction": torch.tensor([-0.9, -0.8, -0.5, -0.6, -0.3, -0.95], dtype=F)}
    ids, w = P.route(torch.ones(2, 6, dtype=F), t, "r.", {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}})
    assert ids.tolist() == [[4, 5], [4, 5]] and torch.allclose(w, torch.full((2, 2), 0.5, dtype=F))
