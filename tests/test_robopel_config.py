"""Robopel on the CPU: its configuration reader, its model description, the
cache it asks for (pooled blocks in pages of their own, layers that read
another layer's keys), the bent rotation tables, and the plain implementation's
own mechanisms against special cases."""

import copy
import math

import pytest
import torch

import nnis_amd
import plain_robopel as R
from nnis_amd.cache import SequenceCache
from nnis_amd.config.registry import spec_from_config
from nnis_amd.errors import CacheFull, InvalidInput, Unsupported
from nnis_amd.models.decoder import DecoderModel
from nnis_amd.parts.base import KVRequest, StateRequest
from nnis_amd.parts.rope import rotary_tables
from robopel_configs import ROB_A, ROB_B, ROB_C, ROBOPEL_CONFIGS, attention, dense, layer, moe, robopel


def test_the_architecture_is_chosen_by_its_name():
    cfg, spec = spec_from_config(ROB_A)
    assert spec.architecture == "Robopel" and spec.width == 96 and spec.vocab_size == 300 and spec.max_positions is None
    assert "Robopel" in nnis_amd.config.registered_architectures()
    assert cfg.embedding_scale == 9.0 and spec_from_config(ROB_B)[0].embedding_scale == 1.0
    with pytest.raises(Unsupported):
        spec_from_config(dict(ROB_A, architecture="Robopel2"))


def test_layers_their_parts_and_whose_keys_they_read():
    for config in (ROB_A, ROB_B, ROB_C):
        _, spec = spec_from_config(config)
        assert [entry.layer for entry in spec.schedule] == list(range(len(config["layers"])))
        for entry, raw, block in zip(spec.schedule, config["layers"], spec.layers):
            assert entry.reads_cache_of == raw["mixer"].get("kv_from")
            assert block["kind"] == "post_norm" and block["norm1"]["offset"] == 1.0
            assert ("feed_forward" in block) == (raw["mlp"] is not None)
            assert block["mixer"]["kind"] == {"attention": "gated_window_attention", "mingru": "min_gru"}[raw["type"]]
            if raw["mlp"] is not None:
                assert block["feed_forward"]["kind"] == {"dense": "poly_norm", "moe": "routed"}[raw["mlp"]["kind"]]
    _, spec = spec_from_config(ROB_A)
    assert len(spec.positions) == 1  # layers 0 and 2 share their bent tables
    names = {t.name: t.shape for t in DecoderModel(spec).tensors()}
    assert "l0.mix.k" in names and "l0.mix.k.norm" in names and "l2.mix.q.norm" in names and names["l2.mix.sink"] == (4,)
    assert not any(name.startswith(("l2.mix.k", "l2.mix.v", "l2.mlp")) for name in names)  # no keys of its own, no feed-forward
    assert names["l1.mlp.router"] == (6, 96) and names["l1.mlp.correction"] == (6,) and names["l1.mlp.e4.down"] == (96, 24)
    assert "l1.mlp.e5.up" not in names and names["l0.mlp.act"] == (4,) and names["l1.mix.z.b"] == (72,)


def test_missing_and_wrong_keys_are_refused():
    for path in (["vocab"], ["norm", "eps"], ["layers", 0, "mixer", "heads"], ["layers", 0, "mixer", "scale"], ["layers", 0, "mixer", "vdim"],
                 ["layers", 0, "mixer", "rot", "base"], ["layers", 0, "mixer", "rot", "scaling", "low"], ["layers", 0, "mixer", "mask", "size"],
                 ["layers", 0, "mlp", "ff"], ["layers", 1, "mixer", "width"], ["layers", 1, "mlp", "router", "top"],
                 ["layers", 1, "mlp", "expert"]):
        raw = copy.deepcopy(ROB_A)
        at = raw
        for key in path[:-1]:
            at = at[key]
        del at[path[-1]]
        with pytest.raises(InvalidInput):
            spec_from_config(raw)
    for change, error in ((lambda raw: raw["layers"][1].update(type="conv"), Unsupported),
                          (lambda raw: raw["layers"][0]["mlp"].update(kind="gated"), Unsupported),
                          (lambda raw: raw["layers"][2]["mixer"].update(kv_from=1), InvalidInput),  # a minGRU keeps no keys
                          (lambda raw: raw["layers"][2]["mixer"].update(kv_from=2), InvalidInput),  # not an earlier layer
                          (lambda raw: raw["layers"][2]["mixer"].update(dim=16), InvalidInput),  # other sizes than the keys it reads
                          (lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=34), InvalidInput),
                          (lambda raw: raw["layers"][0]["mixer"].update(heads=5), InvalidInput),
                          (lambda raw: raw["layers"][1]["mlp"]["router"].update(top=7), InvalidInput)):
        raw = copy.deepcopy(ROB_A)
        change(raw)
        with pytest.raises(error):
            spec_from_config(raw)
    raw = copy.deepcopy(ROB_B)
    raw["layers"].append(layer("attention", attention(3, 1, 16, 48, kv_from=2)))  # layer 2 itself reads layer 1's
    with pytest.raises(InvalidInput):
        spec_from_config(raw)
    raw = copy.deepcopy(ROB_C)
    del raw["layers"][0]["mixer"]["mask"]["size"]
    with pytest.raises(InvalidInput):
        spec_from_config(raw)


def test_what_the_file_does_not_mention_does_not_exist():
    bare = robopel(vocab=50, width=32, layers=[{"type": "mingru", "mixer": {"width": 8}}])  # no "mlp" at all: no feed-forward
    assert "feed_forward" not in spec_from_config(bare)[1].layers[0]
    zeros = robopel(vocab=50, width=32, layers=[layer("attention", dict(attention(2, 1, 16, 8, window=5), softcap=0, mask={"size": 5, "pool": 0}))])
    assert (spec_from_config(zeros)[0].layers[0].attention.softcap, spec_from_config(zeros)[0].layers[0].attention.pool) == (0.0, 0)
    config = robopel(vocab=50, width=32, layers=[layer("attention", attention(2, 1, 16, 8, scale=0.3), moe(3, 2, 8))])
    cfg, spec = spec_from_config(config)
    sizes = cfg.layers[0].attention
    assert (sizes.softcap, sizes.rot_dims, sizes.rot_scaling, sizes.window, sizes.pool, sizes.kv_from) == (0.0, 0, None, 0, 0, None)
    assert cfg.layers[0].router.identity == 0 and not spec.positions
    mixer = spec.layers[0]["mixer"]
    assert mixer["softcap"] is None and mixer["window"] is None and mixer["pool"] is None and mixer["position"] is None
    assert DecoderModel(spec).cache_requests()[0] == [(0, (KVRequest(1, 16, None, 8), None))]


def test_the_cache_it_asks_for():
    """Keys and values in pages; pooled blocks in pages of their own, one entry a block; a layer that reads another's keys
    keeps pooled blocks of its own only where its blocks differ from the other's; a minGRU keeps one 32-bit row."""
    requests, shared = DecoderModel(spec_from_config(ROB_A)[1]).cache_requests()
    assert shared == {2: 0}  # the same blocks of 8: nothing beside
    assert requests == [(0, (KVRequest(2, 32, None, 16), KVRequest(2, 32, None, 16, every=8))), (1, StateRequest((72,))), (3, StateRequest((96,)))]
    requests, shared = DecoderModel(spec_from_config(ROB_B)[1]).cache_requests()
    assert shared == {2: 1} and (2, KVRequest(1, 16, None, 48, every=5)) in requests  # blocks of 5 beside the other's of 24
    requests, shared = DecoderModel(spec_from_config(ROB_C)[1]).cache_requests()
    assert shared == {1: 0, 4: 3}
    assert [index for index, _ in requests] == [0, 2, 3, 4]  # layer 1 sees no pooled blocks; layer 4 keeps blocks of 16 beside full keys
    assert dict(requests)[3] == (KVRequest(2, 24, None, 40), None) and dict(requests)[4] == KVRequest(2, 24, None, 40, every=16)


def test_pooled_pages_follow_the_blocks():
    """A group of one entry for every 3 tokens: a sequence of n tokens holds n // 3 entries, so its pooled pages begin
    at 3, 195, 387 tokens; pages go back when a slot is released or shortened, and are counted before a step."""
    requests = [(0, (KVRequest(1, 8), KVRequest(1, 8, every=3)))]
    cache = SequenceCache(requests, {1: 0}, max_tokens=64 * 6, max_positions=64 * 6, dtype=torch.float32, device="cpu")
    main, pooled = cache.kv_groups
    assert pooled.request.every == 3 and cache.bytes_per_token() == main.bytes_per_token() + main.bytes_per_token() // 3
    slot = cache.acquire()
    cache.grow({slot: 2})
    assert len(main.table.rows[slot]) == 1 and len(pooled.table.rows.get(slot, [])) == 0
    cache.grow({slot: 1})
    assert len(pooled.table.rows[slot]) == 1
    cache.grow({slot: 191})  # 194 tokens: 64 whole blocks
    assert len(main.table.rows[slot]) == 4 and len(pooled.table.rows[slot]) == 1
    before, crossing = cache.check_one_more([slot])
    assert before == [194] and crossing == {slot: 1}  # the 195th token completes block 64, which opens a pooled page
    cache.grow_by_one([slot])
    assert len(pooled.table.rows[slot]) == 2 and int(pooled.block_table_host[slot, 1]) == pooled.table.rows[slot][1]
    assert cache.check_one_more([slot])[1] == {}
    view, reading = cache.view(0), cache.view(1)
    assert view[1].block_table is pooled.block_table and not view[1].read_only and reading[1].read_only and reading[0].read_only
    cache.truncate(slot, 100)
    assert len(main.table.rows[slot]) == 2 and len(pooled.table.rows[slot]) == 1
    other = cache.acquire()
    with pytest.raises(CacheFull):
        cache.grow({other: 64 * 5})
    cache.release(slot)
    assert main.table.pool.free == 6 and pooled.table.pool.free == 6
    cache.grow({other: 64 * 6})
    assert len(pooled.table.rows[other]) == 2


def test_pooled_blocks_of_one_token_share_the_keys_pages():
    requests = [(0, (KVRequest(2, 16), KVRequest(2, 16, every=1)))]
    cache = SequenceCache(requests, {}, max_tokens=128, max_positions=128, dtype=torch.float32, device="cpu")
    assert len(cache.kv_groups) == 1 and cache.kv_groups[0].k.shape[0] == 2  # two entries of one group, one block table
    assert cache.view(0)[0].k_pages.data_ptr() != cache.view(0)[1].k_pages.data_ptr()


def test_bent_rotation_tables():
    for dims, base, scaling in ((32, 5000.0, (4.0, 1.0, 2.0, 64)), (24, 1e4, (8.0, 1.0, 4.0, 32)), (8, 100.0, None), (16, 2e4, (8.0, 1.0, 4.0, 512))):
        named = None if scaling is None else dict(zip(("factor", "low", "high", "original"), scaling))
        f = R.scaled_frequencies(dims, base, named)
        cos, sin = rotary_tables(300, dims, base, "float64", scaling)
        angle = torch.arange(300, dtype=torch.float64)[:, None] * f[None, :]
        assert float((cos.double() - torch.cos(angle)).abs().max()) < 1e-6 and float((sin.double() - torch.sin(angle)).abs().max()) < 1e-6
    f = R.scaled_frequencies(32, 5000.0, {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 64})
    plain = torch.tensor([5000.0 ** (-2.0 * i / 32) for i in range(16)], dtype=torch.float64)
    kept, divided = 2 * math.pi / plain < 32, 2 * math.pi / plain > 64
    assert kept.any() and divided.any() and (~kept & ~divided).any()  # all three ranges occur
    assert torch.equal(f[kept], plain[kept]) and torch.allclose(f[divided], plain[divided] / 4.0)
    between = ~kept & ~divided
    assert bool(((f[between] < plain[between]) & (f[between] > plain[between] / 4.0)).all())


def test_the_plain_min_gru_in_special_cases():
    width = 6
    w = {name: torch.zeros(width, width, dtype=torch.float64) for name in ("z", "x")}
    w.update({"g": torch.eye(width, dtype=torch.float64), "o": torch.eye(width, dtype=torch.float64)})
    w["z.b"] = torch.full((width,), 50.0, dtype=torch.float64)  # z = 1: the state is the candidate
    w["x.b"] = torch.tensor([-2.0, -0.5, 0.0, 0.5, 2.0, 7.0], dtype=torch.float64)
    h = torch.ones(3, width, dtype=torch.float64)
    out, state = R.min_gru(h, w)
    candidate = torch.tensor([1 / (1 + math.exp(2.0)), 1 / (1 + math.exp(0.5)), 0.5, 1.0, 2.5, 7.5], dtype=torch.float64)
    assert torch.allclose(state, candidate) and torch.allclose(out[0], candidate * R.silu(h[0]))
    w["z.b"] = torch.zeros(width, dtype=torch.float64)  # z = 1/2: S_t = (S_(t-1) + c) / 2 from zero
    _, state = R.min_gru(h, w)
    assert torch.allclose(state, candidate * (1 - 0.5 ** 3))
    first, carried = R.min_gru(h[:2], w)
    second, state2 = R.min_gru(h[2:], w, state=carried)
    assert torch.allclose(state2, state)  # the state carries a sequence over a cut


def test_the_plain_attention_sees_window_blocks_and_sink():
    """One head, no rotation, queries and keys that make every score equal: the weights are then counts.  With a window
    of 4 and blocks of 3, token 10 sees tokens 7..10, blocks 0 and 1 (tokens 0..5), not token 6, and the sink."""
    dim, n = 4, 11
    sizes = {"heads": 1, "kv_heads": 1, "dim": dim, "vdim": 1, "scale": 1.0, "mask": {"size": 4, "pool": 3}}
    w = {"q": torch.zeros(dim, 2, dtype=torch.float64), "k": torch.zeros(dim, 2, dtype=torch.float64), "v": torch.tensor([[0.0, 1.0]], dtype=torch.float64),
         "q.norm": torch.ones(dim, dtype=torch.float64), "k.norm": torch.ones(dim, dtype=torch.float64), "sink": torch.zeros(1, dtype=torch.float64),
         "g": torch.tensor([[50.0, 0.0]], dtype=torch.float64), "o": torch.ones(1, 1, dtype=torch.float64)}
    h = torch.ones(n, 2, dtype=torch.float64)
    h[:, 1] = torch.arange(n, dtype=torch.float64)  # a token's value is its position
    out, _ = R.pooled_window_attention(h, w, sizes, 1e-5)
    # scores are all 0: 4 tokens, 2 blocks and the sink share the weight; the blocks' values are the means 1 and 4
    assert abs(float(out[10]) - (7 + 8 + 9 + 10 + 1 + 4) / 7.0) < 1e-9
    assert abs(float(out[3]) - (0 + 1 + 2 + 3) / 5.0) < 1e-9  # nothing has left the window yet
    assert abs(float(out[6]) - (3 + 4 + 5 + 6 + 1) / 6.0) < 1e-9  # block 0 (ends at 2 <= 6 - 4) is seen, tokens 0..2 are not
    w["sink"] = torch.full((1,), -50.0, dtype=torch.float64)
    assert abs(float(R.pooled_window_attention(h, w, sizes, 1e-5)[0][10]) - (7 + 8 + 9 + 10 + 1 + 4) / 6.0) < 1e-9


def test_the_plain_router_in_special_cases():
    width, experts = 4, 3
    w = {"router": torch.zeros(experts + 1, width, dtype=torch.float64), "correction": torch.tensor([0.0, 0.0, 1.0, 0.7], dtype=torch.float64)}
    w["router"][:, 0] = torch.tensor([3.0, 2.0, 0.0, 1.0], dtype=torch.float64)
    for e in range(experts):
        w[f"e{e}.up"] = torch.eye(width, dtype=torch.float64) * (e + 1)
        w[f"e{e}.down"] = torch.eye(width, dtype=torch.float64)
    h = torch.tensor([[1.0, -1.0, 2.0, 0.5]], dtype=torch.float64)
    out, chosen = R.routed_feed_forward(h, w, {"experts": experts, "identity": 1, "top": 2})
    s = torch.softmax(torch.tensor([3.0, 2.0, 0.0, 1.0], dtype=torch.float64), dim=0)
    assert sorted(chosen[0].tolist()) == [2, 3]  # the correction lifts the two smallest scores over the others
    want = s[2] * torch.relu(3.0 * h[0]) ** 2 + s[3] * h[0]  # weights without the correction, not renormalised; the identity output hands h on
    assert torch.allclose(out[0], want)


@pytest.mark.parametrize("name", sorted(ROBOPEL_CONFIGS))
def test_the_plain_model_gives_a_prefix_the_same_logits(tmp_path, name):
    config, seed = ROBOPEL_CONFIGS[name]
    folder = str(tmp_path / name)
    nnis_amd.write_random_model(folder, config, seed)
    plain = R.PlainRobopel(folder)
    ids = torch.randint(0, config["vocab"], (90,), generator=torch.Generator().manual_seed(1)).tolist()
    whole, streams = plain.logits(ids), []
    part = plain.logits(ids[:50], stream_after=streams)
    assert torch.allclose(whole[:50], part, atol=1e-9) and len(streams) == len(config["layers"])
    assert plain.greedy(ids[:5], 3) == plain.greedy(ids[:5], 3)
