"""Gonurax without a GPU: its config.json reader and plan, its tensor names, the page manager's kept first keys, and
the plain implementation held against hand-worked values and against itself (whole against portions)."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import gonurax_helpers as gh
import plain_gonurax as plain


def test_config_is_read_key_by_key_and_refuses_what_it_does_not_know():
    from mini_engine_amd.config.registry import architecture_name_of, get_architecture
    from mini_engine_amd.models.gonurax import GonuraxConfig

    cfg = gh.configs()["P"]
    assert architecture_name_of(cfg) == "Gonurax"
    typed = get_architecture("Gonurax").config_from_dict(cfg)
    assert (typed.vocab, typed.width, typed.norm_groups, typed.residual_mult, typed.norm_eps) == (300, 96, 3, 0.5, 1e-5)
    assert GonuraxConfig.from_dict(typed.to_config_json()) == typed
    for path, value in ((("layers", 0, "type"), "mamba"), (("layers", 1, "mixer", "kv_heads"), 3),
                        (("layers", 0, "mixer", "decay"), [0.5]), (("norm", "groups"), 7),
                        (("layers", 0, "mlp", "kind"), "routed"), (("layers", 1, "mixer", "vdim"), 47),
                        (("layers", 0, "mixer", "rot", "dims"), 34)):
        bad = copy.deepcopy(cfg)
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ValueError):
            GonuraxConfig.from_dict(bad)
    lacking = copy.deepcopy(cfg)
    del lacking["layers"][1]["mixer"]["mask"]
    with pytest.raises(ValueError, match="mask"):
        GonuraxConfig.from_dict(lacking)


def test_plan_takes_every_size_and_constant_from_the_config():
    from mini_engine_amd.models.gonurax import GonuraxConfig, plan_from_config
    from mini_engine_amd.parts.decoder import Decoder

    cfg = gh.configs()["P"]
    plan = plan_from_config(GonuraxConfig.from_dict(cfg))
    assert plan.tie_word_embeddings and plan.embed_name == "embed" and plan.final_norm_name == "final.norm"
    assert plan.final_norm.groups == 3 and plan.final_norm.eps == 1e-5
    kinds = [layer.mixer.kind for layer in plan.layers]
    assert kinds == ["decay_state", "attention", "decay_state", "attention"]
    assert all(layer.arrangement == "parallel" and layer.residual_scale == 0.5 for layer in plan.layers)
    ret, att, lit, att2 = (layer.mixer for layer in plan.layers)
    assert (ret.num_heads, ret.key_dim, ret.value_dim, ret.decay) == (3, 32, 16, (0.9, 0.97, 0.995))
    assert ret.key_scale == 32 ** -0.5 and ret.output_norm == "per_head" and ret.gate_activation == "silu"
    assert ret.position.pairing == "halves" and ret.position.rotary_dim == 16
    assert lit.input_activation == "silu" and lit.output_norm == "all_heads" and lit.gate_activation == "sigmoid"
    assert lit.position is None and lit.key_scale == 1.0
    assert (att.num_heads, att.num_kv_heads, att.head_dim, att.v_dim, att.window, att.keep_first, att.scale) == (4, 2, 32, 48, 24, 5, 0.2)
    assert att.position.pairing == "neighbours" and att.position.rotary_dim == 16 and att.value_position.rotary_dim == 48
    assert att2.keep_first == 0 and att2.window == 40 and att2.value_position.theta == 5e5
    assert plan.layers[1].ffn is None and plan.layers[0].ffn.activation == "gelu_tanh"
    wants = Decoder(plan, torch.float32, "cpu").weight_wants()
    assert wants["l1.mix.q.norm"].shape == (32,) and wants["l1.mix.o"].shape == (96, 4 * 48)
    assert wants["l1.mix.v"].shape == (2 * 48, 96) and wants["l2.mix.norm"].shape == (2 * 24,)
    assert wants["l0.mix.g"].shape == (3 * 16, 96) and wants["l0.mlp.down"].shape == (96, 160)
    assert "l1.mlp.gate" not in wants and "l0.mix.norm" not in wants and "head" not in wants
    assert set(n.split(".")[0] for n in wants) == {"embed", "final", "l0", "l1", "l2", "l3"}


def test_layers_group_their_caches_by_need():
    from mini_engine_amd.cache.storage import plan_layout
    from mini_engine_amd.models.gonurax import GonuraxConfig, plan_from_config
    from mini_engine_amd.parts.decoder import Decoder

    dec = Decoder(plan_from_config(GonuraxConfig.from_dict(gh.configs()["P"])), torch.float32, "cpu")
    layout = plan_layout(dec)
    assert [(g.window, g.keep_first) for g in layout.groups] == [(24, 5), (40, 0)]
    assert layout.layer_group == {1: 0, 3: 1}
    assert {r: n.shape for r, n in layout.state_layers.items()} == {0: (3, 32, 16), 2: (2, 16, 24)}


def test_pages_of_kept_first_keys_stay_while_the_window_moves_on():
    from mini_engine_amd.cache.block_manager import BlockManager, GroupSpec

    bm = BlockManager(32, 4, enable_prefix_caching=False, groups=(GroupSpec(window=6, keep_first=5), GroupSpec(window=6)))
    seq = bm.new_sequence(list(range(40)))
    assert bm.try_allocate(seq, 40)
    seq.num_computed_tokens = 40
    bm.release_passed(seq)
    kept, plain_window = seq.block_tables
    # keys 0..4 live in pages 0 and 1; a query at 40 sees keys from 35 on: page 8
    assert [i for i, p in enumerate(kept) if p >= 0] == [0, 1, 8, 9]
    assert [i for i, p in enumerate(plain_window) if p >= 0] == [8, 9]
    with pytest.raises(ValueError):
        BlockManager(8, 4, groups=(GroupSpec(window=0, keep_first=2),))


def test_visible_keys_of_the_window_with_kept_first_tokens():
    assert [j for j in range(12) if plain.visible(11, j, 4, 3)] == [0, 1, 2, 8, 9, 10, 11]
    assert [j for j in range(12) if plain.visible(5, j, 4, 3)] == [0, 1, 2, 3, 4, 5]
    assert [j for j in range(12) if plain.visible(11, j, 4, 0)] == [8, 9, 10, 11]


def test_rotation_pairs_by_hand():
    v = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]], dtype=torch.float64)
    p = torch.tensor([3])
    base, dims = 100.0, 4
    a0, a1 = 3.0, 3.0 * 100.0 ** (-2.0 / 4.0)
    halves = plain.rotate_pairs(v, p, dims, base, "halves")[0, 0]
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
            3 * math.cos(a0) + 1 * math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(halves, torch.tensor(want, dtype=torch.float64), atol=1e-12)
    inter = plain.rotate_pairs(v, p, dims, base, "interleaved")[0, 0]
    want = [1 * math.cos(a0) - 2 * math.sin(a0), 2 * math.cos(a0) + 1 * math.sin(a0),
            3 * math.cos(a1) - 4 * math.sin(a1), 4 * math.cos(a1) + 3 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(inter, torch.tensor(want, dtype=torch.float64), atol=1e-12)
    back = plain.rotate_pairs(inter[None, None], p, dims, base, "interleaved", sign=-1.0)
    assert torch.allclose(back, v, atol=1e-12)


def test_grouped_norm_by_hand():
    x = torch.tensor([[3.0, 4.0, 0.0, 2.0]], dtype=torch.float64)
    w = torch.tensor([1.0, 2.0, 1.0, 0.5])
    got = plain.grouped_rms_norm(x, w, 2, 0.0)
    r0, r1 = math.sqrt(12.5), math.sqrt(2.0)
    assert torch.allclose(got, torch.tensor([[3 / r0, 8 / r0, 0.0, 1 / r1]], dtype=torch.float64), atol=1e-12)
    one = plain.grouped_rms_norm(x, w, 1, 0.0)
    assert torch.allclose(one, x / math.sqrt(29.0 / 4.0) * w.double(), atol=1e-12)


def test_decayed_state_scan_equals_the_weighted_sum_over_the_past():
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(9, 2, 4, generator=g, dtype=torch.float64), torch.randn(9, 2, 4, generator=g, dtype=torch.float64)
    v = torch.randn(9, 2, 3, generator=g, dtype=torch.float64)
    decay = (0.5, 0.9)
    out, state = plain.decayed_state_scan(q, k, v, decay, None)
    for h, lam in enumerate(decay):
        for t in range(9):
            want = sum(lam ** (t - s) * (q[t, h] @ k[s, h]) * v[s, h] for s in range(t + 1))
            assert torch.allclose(out[t, h], want, atol=1e-12)
    first, s1 = plain.decayed_state_scan(q[:4], k[:4], v[:4], decay, None)
    rest, s2 = plain.decayed_state_scan(q[4:], k[4:], v[4:], decay, s1)
    assert torch.allclose(torch.cat((first, rest)), out, atol=1e-12) and torch.allclose(s2, state, atol=1e-12)


@pytest.mark.parametrize("name", ["P", "R"])
def test_plain_whole_equals_plain_in_portions(tmp_path, name):
    cfg = gh.configs()[name]
    w = gh.read_weights(gh.write_folder(str(tmp_path / name), cfg, seed=3))
    g = torch.Generator().manual_seed(5)
    toks = torch.randint(0, cfg["vocab"], (61,), generator=g).tolist()
    whole = plain.forward(cfg, w, toks)[0]
    cut = plain.forward_in_portions(cfg, w, toks, [1, 3, 20, 21, 47])
    assert torch.allclose(whole, cut, atol=1e-9)
    assert len({int(t) for t in whole.argmax(-1)}) > 8
