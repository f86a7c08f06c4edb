"""The plain Goridra implementation against library functions and special cases, and the configuration and plan of
the design, without a GPU."""
import math

import numpy as np
import pytest
import torch

import goridra_helpers as gh
import plain_goridra as pg


def test_layer_norm_and_gelu_are_the_library_ones():
    rng = np.random.default_rng(0)
    x, w, b = rng.standard_normal((5, 33)) * 4 + 9, rng.standard_normal(33), rng.standard_normal(33)
    want = torch.nn.functional.layer_norm(torch.tensor(x), (33,), torch.tensor(w), torch.tensor(b), 1e-5).numpy()
    assert np.max(np.abs(pg.layer_norm(x, w, b, 1e-5) - want)) < 1e-12
    assert np.max(np.abs(pg.gelu_erf(x) - torch.nn.functional.gelu(torch.tensor(x)).numpy())) < 1e-12


def test_chunk_mask():
    vis = pg.chunk_visible(10, 4)
    assert vis[3].tolist() == [True] * 4 + [False] * 6
    assert vis[4].tolist() == [False] * 4 + [True] + [False] * 5          # the first position of a chunk sees itself only
    assert vis[9].tolist() == [False] * 8 + [True] * 2
    assert pg.chunk_visible(6, 100).tolist() == np.tril(np.ones((6, 6), bool)).tolist()


def test_attention_is_the_library_one_under_the_same_mask():
    rng = np.random.default_rng(1)
    T, H, G, D, Dv = 21, 4, 2, 6, 10
    q, k, v = rng.standard_normal((T, H, D)), rng.standard_normal((T, G, D)), rng.standard_normal((T, G, Dv))
    mask = torch.tensor(pg.chunk_visible(T, 8))
    kk = torch.tensor(k).repeat_interleave(H // G, dim=1).transpose(0, 1)
    vv = torch.tensor(v).repeat_interleave(H // G, dim=1).transpose(0, 1)
    want = torch.nn.functional.scaled_dot_product_attention(torch.tensor(q).transpose(0, 1), kk, vv, attn_mask=mask, scale=0.37)
    assert np.max(np.abs(pg.attend(q, k, v, 0.37, 8) - want.transpose(0, 1).reshape(T, -1).numpy())) < 1e-12


def test_rotation_turns_pairs_and_leaves_the_rest():
    v = np.zeros((1, 1, 8))
    v[0, 0, 0], v[0, 0, 6] = 1.0, 5.0
    out = pg.rotate(v, [3], 4, 10000.0)              # pairs (0, 2) and (1, 3); 4..7 pass
    assert np.allclose(out[0, 0, [0, 2]], [math.cos(3.0), math.sin(3.0)])
    assert out[0, 0, 6] == 5.0 and out[0, 0, 1] == 0.0
    a, b = np.random.default_rng(2).standard_normal((2, 1, 1, 8))
    dots = [float(np.sum(pg.rotate(a, [p + 5], 8, 100.0) * pg.rotate(b, [p], 8, 100.0))) for p in (0, 40)]
    assert abs(dots[0] - dots[1]) < 1e-12            # scores depend on the distance only


def test_router_groups_and_weights():
    z = np.array([[5.0, -9.0, -9.0, -9.0, -9.0, 4.0, 4.1, 3.9, -9.0, -9.0]])
    ids, w = pg.route(z, 3, 2, 1)
    assert ids.tolist() == [[0, 1, 2]] and abs(w.sum() - 1.0) < 1e-12
    ids, w = pg.route(z, 3, 2, 2)
    assert ids.tolist() == [[0, 6, 5]]
    s = pg.softmax(z)[0]
    assert np.allclose(w[0], s[[0, 6, 5]] / s[[0, 6, 5]].sum())
    assert gh.choice_margin(s, 3, 2, 2) == pytest.approx(s[5] - s[7])


def test_a_layer_that_reads_another_layers_keys_and_values_and_a_layer_without_feed_forward(tmp_path):
    cfg = gh.SMALL
    w = gh.make_weights(cfg, 1)
    toks = [3, 200, 17, 5, 99, 250, 1, 1, 42]
    base = pg.forward(cfg, {k: v.astype(np.float64) for k, v in w.items()}, toks)
    assert base.shape == (9, cfg["vocab"]) and np.max(np.abs(base)) < cfg["logit_softcap"]
    # layer 1 has no k and v: changing layer 0's changes it; positions beyond a chunk of layer 3 (7 tokens) do not
    # see its first tokens in that layer, but do through the others
    assert "l1.mix.k" not in w and "l2.mlp.up" not in w
    w2 = dict(w)
    w2["l0.mix.v"] = w["l0.mix.v"] * 0.5
    assert np.max(np.abs(pg.forward(cfg, {k: v.astype(np.float64) for k, v in w2.items()}, toks) - base)) > 1e-3


def test_configuration_and_plan():
    import hf_cpu_amd
    from hf_cpu_amd.config import config_from_dict
    from hf_cpu_amd.model import Model
    from hf_cpu_amd.status import EngineError
    cfg = config_from_dict(gh.SMALL)
    assert cfg.layers[1].mixer.kv_from == 0 and cfg.layers[2].mlp is None and cfg.layers[3].mlp.experts == 5
    model = Model.from_config(cfg)
    names = {s.name: tuple(s.shape) for s in model.param_specs() if not s.optional}
    assert set(names) == set(gh.make_weights(gh.SMALL, 0))
    assert names["l0.mix.v"] == (40, 48) and names["l1.mlp.e5.down"] == (48, 40) and "l1.mix.k" not in names
    needs = model.cache_needs()
    assert needs[1] is None and needs[0].k_width == 24 and needs[0].v_width == 40 and needs[2].k_width == 48
    assert [e.cache_of for e in model.schedule] == [None, 0, None, None]
    for key, value in (("kv_from", 1), ("kv_from", 2)):
        bad = {**gh.SMALL, "layers": [dict(l, mixer=dict(l["mixer"])) for l in gh.SMALL["layers"]]}
        bad["layers"][3]["mixer"][key] = value            # a reader of a reader; a source with other sizes
        with pytest.raises(EngineError):
            config_from_dict(bad)
    bad = {**gh.SMALL, "layers": [dict(gh.SMALL["layers"][0], type="recurrent")]}
    with pytest.raises(EngineError):
        config_from_dict(bad)


def test_pages_before_the_current_chunk_go_back_unless_a_reader_still_sees_them():
    from hf_cpu_amd.cache import CacheManager
    from hf_cpu_amd.parts.base import PagedKV
    need = PagedKV(8, 8, 0, 24, readers=((0, 16),))
    assert [need.first_kept(p) for p in (0, 15, 16, 23, 24, 31, 32, 47, 48, 50)] == [0, 0, 0, 0, 16, 16, 24, 24, 48, 48]
    assert PagedKV(8, 8, 0, 24, readers=((0, 0),)).first_kept(1000) == 0          # a reader that sees everything keeps everything
    assert PagedKV(8, 8, 30, 0, readers=((0, 16),)).first_kept(100) == 71         # a window and a reader's chunk: the earlier of the two
    m = CacheManager([need, None], page_tokens=8, n_pages=7, n_slots=1, max_context=400)
    m.admit("a")
    at = 0
    for n in [10, 3, 9, 1, 1, 7, 10, 2] * 7:
        m.reserve("a", n)
        m.commit("a", n)
        at += n
        table = m.held["a"].tables[0]
        first = need.first_kept(at) // 8
        assert all(p < 0 for p in table[:first]) and all(p >= 0 for p in table[first:])
        m.check()
    assert at > 7 * 8 * 5 and m.pools[0].reused > 0
    m.release("a")
    assert m.pools[0].n_held == 0
