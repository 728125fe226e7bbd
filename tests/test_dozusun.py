"""Dozusun without a GPU: its configuration, plan, checkpoint names and caches, and the plain implementation
held against itself (what a position may depend on, where a window ends, how a stretch of layers repeats)."""

import pytest
import torch

from tests import plain_dozusun as plain
from tests.dozusun_cases import CASES, random_weights


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
    assert arch.name == "Dozusun" and arch.parse_config(config.to_dict()) == config
    assert [r.layer for r in model.plan.run] == plain.run_order(raw) == config.run_order()
    weights = random_weights(raw, seed=1)
    shapes = arch.checkpoint_shapes(config)
    assert set(shapes) == set(weights) and all(tuple(weights[k].shape) == tuple(v[0]) for k, v in shapes.items())
    from atomserve_amd.weights.loader import as_stack

    used = {t.name for target in model.weight_decls() for t in as_stack(arch.checkpoint_map(config)[target]).parts}
    assert used == set(weights), "every tensor of the checkpoint is read, and nothing else is asked for"


def test_every_run_of_a_repeated_layer_has_caches_of_its_own():
    from atomserve_amd.cache.manager import CacheManager
    from atomserve_amd.parts.base import PagedCacheRequest

    raw = CASES["looped"]
    _, config, model = parts_of(raw)
    requests = model.cache_requests()
    runs = len(config.run_order())
    assert {cid[0] for cid in requests} == set(range(runs))
    paged = [cid for cid, req in requests.items() if isinstance(req, PagedCacheRequest)]
    assert paged == [(0, "pages")] and requests[(0, "pages")].window == 9
    manager = CacheManager(requests, 16, 8, 2)
    assert not manager.prefix_reuse_possible and manager.names_of_cache[0] == ["pages", "state", "conv"]
    assert manager.names_of_cache[2] == ["state"]  # a convolution of one tap keeps no inputs
    rc = manager.new_request()
    assert manager.reserve(rc, 0, 40) and rc.state_slot >= 0 and len(rc.tables[0]) == 3
    assert manager.release_behind_window(rc, 40) == 2  # positions 0..31 lie behind a window of 9 at position 40
    manager.release(rc)
    assert manager.num_free == 8 and manager.num_free_slots == 2


def test_what_the_configuration_refuses():
    from atomserve_amd.config.model_config import ConfigError, DozusunConfig

    raw = CASES["plain_order"]
    for change, needle in (
        (lambda r: r["layers"][0].update(type="conv"), "type"),
        (lambda r: r["layers"][0]["mlp"].update(kind="sparse"), "kind"),
        (lambda r: r["layers"][1]["mixer"]["right"].update(blocks=3), "blocks"),
        (lambda r: r["layers"][0]["mixer"].pop("conv"), "conv"),
        (lambda r: r.update(loop={"start": 2, "stop": 5, "times": 2}), "loop"),
        (lambda r: r["layers"][0]["mlp"]["router"].update(top=4), "top"),
    ):
        import copy

        bad = copy.deepcopy(raw)
        change(bad)
        with pytest.raises(ConfigError, match=needle):
            DozusunConfig.from_dict(bad)


def test_random_checkpoints_name_distinct_experts():
    from atomserve_amd.weights.random_init import random_checkpoint

    arch, config, _ = parts_of(CASES["looped"])
    tensors = random_checkpoint(arch, config, seed=4)
    table = tensors["l0.mlp.table"]
    assert table.dtype == torch.int32 and table.shape == (300, 2) and int(table.min()) >= 0 and int(table.max()) < 5
    assert bool((table[:, 0] != table[:, 1]).all())


# ---- the plain implementation against itself ------------------------------------------------------------


def test_plain_a_position_depends_on_nothing_after_it_and_on_everything_before():
    raw = CASES["looped"]
    w = random_weights(raw, seed=2)
    ids = torch.randint(0, raw["vocab"], (30,), generator=torch.Generator().manual_seed(0)).tolist()
    full = plain.logits(raw, w, ids)
    assert torch.allclose(plain.logits(raw, w, ids[:17]), full[:17], atol=1e-6)
    other = list(ids)
    other[0] = (ids[0] + 1) % raw["vocab"]
    assert (plain.logits(raw, w, other)[-1] - full[-1]).abs().max() > 1e-4  # the states carry the first token to the end


def test_plain_window_and_convolution_edges():
    T = 12
    gen = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(T, 1, 4, generator=gen, dtype=torch.float64) for _ in range(3))
    out = plain.windowed_attention(q, k, v, 0.5, 3)
    for i in range(T):
        lo = max(0, i - 2)
        s = torch.softmax((k[lo : i + 1, 0] @ q[i, 0]) * 0.5, 0)
        assert torch.allclose(out[i, 0], s @ v[lo : i + 1, 0])
    assert torch.allclose(plain.windowed_attention(q, k, v, 0.5, 1)[:, 0], v[:, 0])  # a window of one sees itself only
    assert torch.allclose(plain.windowed_attention(q, k, v, 0.5, 0), plain.windowed_attention(q, k, v, 0.5, T))
    x = torch.randn(T, 3, generator=gen, dtype=torch.float64)
    w = torch.randn(3, 4, generator=gen, dtype=torch.float64)
    y = plain.short_conv(x, w)
    assert torch.allclose(y[0], w[:, 3] * x[0]) and torch.allclose(y[5], sum(w[:, j] * x[5 - (3 - j)] for j in range(4)))


def test_plain_delta_rule_reads_back_what_it_wrote():
    """With no decay, beta = 1 and orthonormal keys the state returns each key's value exactly."""
    D, Dv = 4, 3
    keys = torch.eye(D, dtype=torch.float64)
    values = torch.randn(D, Dv, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    S = torch.zeros(D, Dv, dtype=torch.float64)
    for t in range(D):
        u = 1.0 * (values[t] - S.T @ keys[t])
        S = S + torch.outer(keys[t], u)
    assert torch.allclose(S.T @ keys[1], values[1])
