"""Koravik without a GPU: its configuration, plan, checkpoint names and caches, and the plain implementation
held against itself (what a position may see, what mixing the heads and gating the sums do, how a stretch of
layers repeats and re-enters)."""

import copy

import pytest
import torch

from tests import plain_koravik as plain
from tests.koravik_cases import CASES, random_weights


def parts_of(raw):
    from atomserve_amd.config.registry import architecture_for
    from atomserve_amd.models.decoder import DecoderModel

    arch = architecture_for(raw)
    config = arch.parse_config(raw)
    return arch, config, DecoderModel(arch.build_plan(config), torch.float32, "cpu")


@pytest.mark.parametrize("case", sorted(CASES))
def test_configuration_plan_and_names(case):
    raw = CASES[case]
    arch, config, model = parts_of(raw)
    assert arch.name == "Koravik" and arch.parse_config(config.to_dict()) == config
    assert [(r.layer, r.reenter) for r in model.plan.run] == plain.run_order(raw) == config.run_order()
    assert model.plan.tied_head and model.plan.logit_scale == raw["logit_scale"] and model.plan.embed_norm is not None
    weights = random_weights(raw, seed=1)
    shapes = arch.checkpoint_shapes(config)
    assert set(shapes) == set(weights) and all(tuple(weights[k].shape) == tuple(v[0]) for k, v in shapes.items())
    from atomserve_amd.weights.loader import as_stack

    used = {t.name for target in model.weight_decls() for t in as_stack(arch.checkpoint_map(config)[target]).parts}
    assert used == set(weights), "every tensor of the checkpoint is read, and nothing else is asked for"
    assert model.capturable


def test_runs_have_caches_of_their_own_and_kept_tokens_keep_their_pages():
    from atomserve_amd.cache.manager import RELEASED, CacheManager

    raw = CASES["looped"]
    _, config, model = parts_of(raw)
    requests = model.cache_requests()
    assert sorted(requests) == list(range(len(config.run_order()))) == list(range(7))
    assert (requests[0].window, requests[0].keep_first) == (9, 3) and (requests[2].window, requests[2].keep_first) == (5, 7)
    assert requests[1] == requests[3] == requests[5] and requests[1].keep_first == 0
    manager = CacheManager(requests, 4, 40, 2)
    assert not manager.prefix_reuse_possible and len(manager.paged_groups) == 3
    rc = manager.new_request()
    assert manager.reserve(rc, 0, 40) and all(len(t) == 10 for t in rc.tables)
    manager.release_behind_window(rc, 40)
    by_window = {g.window: t for g, t in zip(manager.paged_groups, rc.tables)}
    # window 9, 3 kept: page 0 stays, positions 4..31 are gone; window 21, none kept: 0..19 gone;
    # window 5, 7 kept: pages 0 and 1 stay, positions 8..35 are gone
    assert [p == RELEASED for p in by_window[9]] == [False] + [True] * 7 + [False] * 2
    assert [p == RELEASED for p in by_window[21]] == [True] * 5 + [False] * 5
    assert [p == RELEASED for p in by_window[5]] == [False] * 2 + [True] * 7 + [False]
    manager.release(rc)
    assert manager.num_free == 40


def test_what_the_configuration_refuses():
    from atomserve_amd.config.model_config import ConfigError, KoravikConfig

    raw = CASES["looped"]
    for change, needle in (
        (lambda r: r["layers"][0].update(type="delta"), "type"),
        (lambda r: r["layers"][0]["mlp"].update(kind="dense"), "kind"),
        (lambda r: r["layers"][0]["mixer"].update(vdim=8), "vdim"),
        (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
        (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
        (lambda r: r["layers"][0]["mixer"].pop("scale"), "scale"),
        (lambda r: r["layers"][0]["mixer"]["mask"].update(size=-1), "mask.size"),
        (lambda r: r["layers"][1]["mixer"].update(kv_heads=2), "kv_heads"),
        (lambda r: r.update(loop={"start": 2, "stop": 5, "times": 2}), "loop"),
        (lambda r: r["layers"][0]["mlp"]["router"].update(top=6), "top"),
        (lambda r: r.pop("residual_mult"), "residual_mult"),
    ):
        bad = copy.deepcopy(raw)
        change(bad)
        with pytest.raises(ConfigError, match=needle):
            KoravikConfig.from_dict(bad)


def test_a_mixer_without_a_mask_or_a_rotation_sees_every_earlier_key_and_turns_nothing():
    from atomserve_amd.config.model_config import KoravikConfig

    raw = copy.deepcopy(CASES["wide_groups"])
    raw["layers"][0]["mixer"].pop("mask")
    raw["layers"][1]["mixer"].pop("rot")
    config = KoravikConfig.from_dict(raw)
    assert (config.layers[0].mixer.window, config.layers[0].mixer.keep_first, config.layers[1].mixer.rot_dims) == (0, 0, 0)
    assert KoravikConfig.from_dict(config.to_dict()) == config
    _, _, model = parts_of(raw)
    assert model.cache_requests()[0].window == 0 and model.blocks[1].parts()["mixer"].position is None


def test_a_layer_with_gated_sums_needs_parts_that_compute_their_gate():
    from atomserve_amd.parts.base import BuildEnv, build
    from atomserve_amd.parts.plan import BlockSpec, MixedHeadsAttentionSpec, NormSpec

    env = BuildEnv(torch.float32, torch.device("cpu"))
    mixer = MixedHeadsAttentionSpec("mixed_heads_attention", 32, 2, 1, 8, 0.3, None, out_gate=False)
    with pytest.raises(ValueError, match="out_gate"):
        build("arrangement", BlockSpec("gated_prenorm", mixer, NormSpec("rmsnorm", 32, 1e-6), None, None), env)
    part = build("mixer", MixedHeadsAttentionSpec("mixed_heads_attention", 32, 2, 1, 12, 0.3, None, window=5, keep_first=2,
                                                 values="own", out_gate=True), env)  # fmt: skip
    assert part.weight_decls()["in.weight"].shape == ((2 + 1 + 1) * 12 + 32, 32) and part.padded_dim == 16
    assert part.cache_request().keep_first == 2 and part.cache_request().head_dim == 16
    with pytest.raises(ValueError, match="heads"):
        build("mixer", MixedHeadsAttentionSpec("mixed_heads_attention", 32, 3, 2, 8, 0.3, None), env)


def test_random_checkpoints_mix_heads_around_the_identity():
    from atomserve_amd.weights.random_init import random_checkpoint

    arch, config, _ = parts_of(CASES["wide_groups"])
    tensors = random_checkpoint(arch, config, seed=4, dtype=torch.float32)
    talk = tensors["l1.mix.talk"]
    assert talk.shape == (18, 18) and float(talk.diagonal().mean()) > 0.7 and float((talk - torch.eye(18)).abs().mean()) < 0.4
    assert "loop.in" in tensors and "l1.mlp.shared.up" in tensors and "l0.mlp.shared.up" not in tensors


# ---- the plain implementation against itself ------------------------------------------------------------


def test_plain_what_a_position_sees():
    seen = plain.visible(12, 4, 2)
    for i in range(12):
        for j in range(12):
            assert bool(seen[i, j]) == (j <= i and (i - j < 4 or j < 2))
    assert bool(plain.visible(6, 1, 0).diagonal().all()) and int(plain.visible(6, 1, 0).sum()) == 6
    assert torch.equal(plain.visible(7, 100, 0), torch.ones(7, 7, dtype=torch.bool).tril())


def test_plain_mixing_the_heads_by_the_identity_is_plain_attention_and_a_swap_swaps_them():
    gen = torch.Generator().manual_seed(3)
    T, H, G, D = 9, 4, 2, 6
    q = torch.randn(T, H, D, generator=gen, dtype=torch.float64)
    k = torch.randn(T, G, D, generator=gen, dtype=torch.float64)
    v = torch.randn(T, G, D, generator=gen, dtype=torch.float64)
    base = plain.mixed_softmax_attention(q, k, v, None, 0.4, 5, 1)
    assert torch.allclose(base, plain.mixed_softmax_attention(q, k, v, torch.eye(H), 0.4, 5, 1))
    for i in range(T):  # against the definition, position by position
        for h in range(H):
            js = [j for j in range(i + 1) if i - j < 5 or j < 1]
            s = torch.softmax(torch.stack([q[i, h] @ k[j, h // 2] * 0.4 for j in js]), 0)
            assert torch.allclose(base[i, h], sum(a * v[j, h // 2] for a, j in zip(s, js)))
    swap = torch.eye(H)[[1, 0, 2, 3]]  # head 0 takes head 1's scores and the other way round; both read kv head 0
    swapped = plain.mixed_softmax_attention(q, k, v, swap, 0.4, 5, 1)
    assert torch.allclose(swapped[:, 0], base[:, 1]) and torch.allclose(swapped[:, 1], base[:, 0])
    assert torch.allclose(swapped[:, 2:], base[:, 2:])


def test_plain_turning_is_a_rotation_of_pairs_and_leaves_the_rest():
    gen = torch.Generator().manual_seed(4)
    x = torch.randn(5, 2, 10, generator=gen, dtype=torch.float64)
    y = plain.turn_half(x, torch.arange(5), 6, 100.0)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0])
    assert torch.allclose((y[..., :6] ** 2).sum(-1), (x[..., :6] ** 2).sum(-1))
    a = 3 * 100.0 ** (-2.0 / 6)  # position 3, pair (1, 4)
    assert torch.allclose(y[3, 0, 1], x[3, 0, 1] * torch.cos(torch.tensor(a)) - x[3, 0, 4] * torch.sin(torch.tensor(a)))
    assert torch.allclose(y[3, 0, 4], x[3, 0, 4] * torch.cos(torch.tensor(a)) + x[3, 0, 1] * torch.sin(torch.tensor(a)))


def test_plain_routing_weighs_the_chosen_by_their_scores():
    h = torch.tensor([[1.0, 0.0], [0.0, 2.0]], dtype=torch.float64)
    router = torch.tensor([[3.0, -1.0], [1.0, 1.0], [-2.0, 0.5]], dtype=torch.float64)
    chosen, weights = plain.route(h, router, 2)
    s = torch.sigmoid(h @ router.T)
    assert chosen.tolist() == [[0, 1], [1, 2]]
    assert torch.allclose(weights[0], s[0, [0, 1]] / s[0, [0, 1]].sum()) and torch.allclose(weights.sum(-1), torch.ones(2, dtype=torch.float64))


def test_plain_a_position_depends_on_the_kept_tokens_and_its_window_only():
    raw = copy.deepcopy(CASES["plain_order"])
    raw["layers"] = raw["layers"][2:]  # one layer: window 6, one token kept, no feed-forward
    w = random_weights(raw, seed=2)
    ids = torch.randint(0, raw["vocab"], (30,), generator=torch.Generator().manual_seed(0)).tolist()
    full = plain.logits(raw, w, ids)
    assert torch.allclose(plain.logits(raw, w, ids[:17]), full[:17], atol=1e-6)
    for place, matters in ((0, True), (1, False), (23, False), (24, True)):  # the last position sees 0 and 24..29
        other = list(ids)
        other[place] = (ids[place] + 1) % raw["vocab"]
        changed = float((plain.logits(raw, w, other)[-1] - full[-1]).abs().max())
        assert (changed > 1e-7) == matters, (place, changed)  # what is not seen changes nothing at all


def test_plain_a_stretch_that_repeats_enters_through_its_matrix_every_time():
    raw = CASES["looped"]
    w = {k: v.double() for k, v in random_weights(raw, seed=5).items()}
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    layers = []
    plain.forward(ids, raw, w, layers_out=layers)
    assert len(layers) == 7
    x0 = plain.rms_norm(w["embed"][torch.tensor(ids)], w["embed.norm"], raw["norm"]["eps"])
    x = torch.cat([layers[2], x0], -1) @ w["loop.in"].T  # the second pass starts from the first pass's end
    x = plain.layer(x, 1, raw, w)
    assert torch.allclose(x, layers[3])
    silent = dict(w)
    silent["loop.in"] = torch.cat([torch.eye(96), torch.zeros(96, 96)], 1).double()  # the stream passes, x0 is not read
    a = plain.forward(ids, raw, silent)
    flat = copy.deepcopy(raw)
    flat["layers"] = [raw["layers"][i] for i in (0, 1, 2, 1, 2, 1, 2)]
    flat.pop("loop")
    renamed = {k: v for k, v in silent.items() if not k.startswith("l")}
    for new, old in enumerate((0, 1, 2, 1, 2, 1, 2)):
        renamed.update({f"l{new}." + k.split(".", 1)[1]: v for k, v in silent.items() if k.startswith(f"l{old}.")})
    assert torch.allclose(a, plain.forward(ids, flat, renamed))
