"""Reading a Dokulix config.json, the parts it becomes, the order its layers run in, the tensor
names, and the cache bookkeeping of blocks of positions and latent rows; no GPU."""
import copy

import pytest
import torch

from rocml_amd.cache import Cache
from rocml_amd.config import architecture_of
from rocml_amd.config.dokulix import DokulixConfig, checkpoint_names, distance_slopes
from rocml_amd.engine.model import DecoderModel
from rocml_amd.errors import ConfigError
from rocml_amd.parts.base import KVCacheRequest, LatentCacheRequest
from tests import dokulix_models as dm
from tests.plain import dokulix_plain as plain


def test_architecture_is_found_by_its_name_and_round_trips():
    arch = architecture_of(dm.CFG_P)
    assert arch.name == "Dokulix"
    cfg = arch.read_config(dm.CFG_P)
    assert DokulixConfig.from_dict(cfg.to_dict()) == cfg
    assert cfg.to_dict() == dm.CFG_P


@pytest.mark.parametrize("name", ["P", "Q", "R"])
def test_run_order_offsets_and_tensor_names(name):
    raw, _ = dm.CONFIGS[name]
    cfg = DokulixConfig.from_dict(raw)
    spec = cfg.to_model_spec()
    assert [(e.layer, e.offset_row) for e in spec.schedule] == plain.layer_order(raw)
    assert spec.pass_offsets == (raw["loop"]["times"] if raw.get("loop") else 0)
    model = DecoderModel(spec, torch.float32, device="meta")
    names = checkpoint_names(spec)
    shapes = dm.tensor_shapes(raw)
    params = model.param_specs()
    assert {names[k]: tuple(p.shape) for k, p in params.items()} == shapes
    # every execution of a looped layer has a cache line of its own
    requests = model.cache_requests()
    assert len(requests) == len(spec.schedule) and all(r is not None for r in requests)


def test_parts_take_their_constants_from_the_configuration():
    spec = DokulixConfig.from_dict(dm.CFG_P).to_model_spec()
    lat, att, lat2, att2 = (b.mixer for b in spec.layers)
    assert (lat.window, lat.kv_rank, lat.rot_dim, lat.position.rot_dim, lat.position.theta) == (20, 40, 8, 8, 100.0)
    assert (lat2.rot_dim, lat2.position.rot_dim) == (16, 8)
    assert (att.chunk, att.window, att.v_head_dim, att.sink, att.bias) == (24, None, 16, True, True)
    assert att.distance_slopes == distance_slopes(4) and att.distance_slopes[3] == 2.0 ** -8
    assert att2.scale == 0.4
    assert spec.layers[2].ffn is None and spec.layers[2].ffn_norm is None
    assert spec.layers[0].mixer_norm.unit_offset and spec.final_norm.unit_offset and not lat.q_norm.unit_offset
    assert spec.layers[0].ffn.activation == "relu"


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="mamba"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), "dims"),
    (lambda c: c["layers"][0].update(mlp={"kind": "routed", "ff": 8}), "mlp"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_bad_configurations_are_refused_with_the_key_named(change, word):
    raw = copy.deepcopy(dm.CFG_P)
    change(raw)
    with pytest.raises(ConfigError, match=word):
        DokulixConfig.from_dict(raw).to_model_spec()


def test_blocks_give_their_pages_back_at_block_borders():
    requests = [KVCacheRequest(2, 8, None, v_head_dim=4, chunk=100), LatentCacheRequest(12, window=70), KVCacheRequest(2, 8)]
    cache = Cache(requests, max_tokens=64 * 40, dtype=torch.float32, device="cpu")
    blocks, latent, kept = cache.kv_groups
    assert (blocks.chunk, latent.window, kept.span) == (100, 70, None)
    assert latent.k.shape[2:] == (64, 12) and blocks.v.shape[2:] == (2, 4, 64)
    slot = cache.new_sequence()
    for length in (64, 99, 100, 199, 200, 256, 300, 301):
        cache.reserve([slot], [length])
        cache.commit([slot], [length])
        # the next query sits at position `length`: it looks back to the start of its block / over its window
        first_block = (length - length % 100) // 64
        first_window = max(0, length - 70 + 1) // 64
        assert [p >= 0 for p in blocks.page_table(slot)] == [i >= first_block for i in range(len(blocks.page_table(slot)))]
        assert [p >= 0 for p in latent.page_table(slot)] == [i >= first_window for i in range(len(latent.page_table(slot)))]
        assert all(p >= 0 for p in kept.page_table(slot))
        cache.check()
    cache.free_sequence(slot)
    assert all(g.n_free_pages == g.n_pages for g in cache.kv_groups)


def test_groups_with_blocks_are_sized_for_a_block():
    requests = [KVCacheRequest(2, 8, None, chunk=100), LatentCacheRequest(12, window=70)]
    cache = Cache(requests, max_tokens=64 * 1000, dtype=torch.float32, device="cpu", max_seqs=2, step_tokens=128)
    assert [g.n_pages for g in cache.kv_groups] == [2 * (2 + 2) + 2, 2 * (2 + 2) + 2]
    assert cache.fits([[("a", 128)], [("a", 256)], [("a", 384)]], final=[("a", 5000)]) is None
