"""What of the Gadopel design needs no GPU: the configuration reader, the model as data (run
order of looped layers, tensor names, the model folder the random-weights mode writes), the
frequency rule, the cache manager's window groups that keep a request's first pages, and pins of
the plain implementation against other formulations."""
import copy
import math

import numpy as np
import pytest
import torch

import gadopel_util as U
import plain_gadopel as plain
from kv_cache_optimization_for_llm_amd.cache.manager import CacheManager
from kv_cache_optimization_for_llm_amd.config.model_config import ConfigError
from kv_cache_optimization_for_llm_amd.models.builder import spec_for_config, tensor_specs_for_config
from kv_cache_optimization_for_llm_amd.parts.base import attention_cache_spec
from kv_cache_optimization_for_llm_amd.parts.latent_attention import latent_cache_spec
from kv_cache_optimization_for_llm_amd.parts.rotary import yarn_frequencies, yarn_magnitude


def test_run_order_repeats_the_looped_layers_with_caches_of_their_own():
    _, spec = spec_for_config(U.CFG_R)
    assert [(c.layer, c.before) for c in spec.order] == [(0, None), (1, 0), (2, None), (1, 0), (2, None), (3, None)]
    assert [c.cache for c in spec.order] == list(range(6))
    _, spec = spec_for_config(U.CFG_P)               # the loop starts at the first layer
    assert [(c.layer, c.before) for c in spec.order] == [(0, 0), (1, None)] * 3 + [(2, None)]
    _, spec = spec_for_config(U.CFG_Q)               # no loop: no operation between layers, no tensor for one
    assert spec.stream_ops == () and all(c.before is None for c in spec.order)
    assert "loop.in" not in tensor_specs_for_config(U.CFG_Q)
    assert spec.residual_dtype == "float32"


def test_tensor_names_and_shapes_follow_the_configuration():
    specs = tensor_specs_for_config(U.CFG_P)
    W = 96
    want = {"embed": (211, W), "head": (211, W), "final.norm": (W,), "loop.in": (W, 2 * W),
            "l0.norm1": (W,), "l0.norm2": (W,), "l0.mix.q": (4 * 32, W), "l0.mix.k": (2 * 32, W),
            "l0.mix.v": (2 * 16, W), "l0.mix.o": (W, 4 * 16), "l0.mlp.gate": (160, W), "l0.mlp.up": (160, W),
            "l0.mlp.down": (W, 160),
            "l1.norm1": (W,), "l1.mix.q": (3 * (16 + 8), W), "l1.mix.dkv": (40 + 8, W), "l1.mix.dkv.norm": (40,),
            "l1.mix.uk": (3 * 16, 40), "l1.mix.uv": (3 * 24, 40), "l1.mix.sink": (3,), "l1.mix.g": (3, W),
            "l1.mix.o": (W, 3 * 24)}
    for name, shape in want.items():
        assert tuple(specs[name].shape) == shape, name
    assert "l1.norm2" not in specs and "l1.mlp.gate" not in specs       # a layer without a feed-forward
    assert "l2.norm2" in specs


@pytest.mark.parametrize("change, message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=6), "rot_dim"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=40), "exceeds"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "kind"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_a_configuration_that_cannot_run_is_refused(change, message):
    cfg = copy.deepcopy(U.CFG_P)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        spec_for_config(cfg)


def test_random_weights_mode_writes_a_folder_the_plain_model_reads(tmp_path):
    folder, state = U.write_model(str(tmp_path / "m"), U.CFG_Q, 3)
    from safetensors.torch import load_file
    stored = load_file(folder + "/model.safetensors")
    assert set(stored) == set(tensor_specs_for_config(U.CFG_Q))
    logits = plain.forward(U.CFG_Q, stored, U.prompt(U.CFG_Q, 12, 0))
    assert logits.shape == (12, 157) and torch.isfinite(logits).all()


def test_yarn_frequencies_and_magnitude():
    for dims, base, sc in [(64, 300000.0, dict(factor=6.0, original=1024, fast=24.0, slow=2.0)),
                           (16, 10000.0, dict(factor=4.0, original=64, fast=8.0, slow=2.0)),
                           (8, 10000.0, dict(factor=16.0, original=32, fast=4.0, slow=1.0))]:
        got = yarn_frequencies(dims, base, **sc)
        want, mag = plain.rotary_frequencies(dims, base, sc)
        np.testing.assert_allclose(got, np.array(want), rtol=1e-14)
        assert yarn_magnitude(sc["factor"]) == pytest.approx(mag)
        plain_f = np.array(plain.rotary_frequencies(dims, base)[0])
        assert (got <= plain_f * (1 + 1e-12)).all() and (got >= plain_f / sc["factor"] * (1 - 1e-12)).all()
        assert got[0] == pytest.approx(plain_f[0])          # the fastest pair keeps its frequency
    # pair indices of the two turn counts, by hand: dims 16, base 1e4, original 64
    index = lambda t: 16 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(1e4))
    assert math.floor(index(8.0)) == 0 and math.ceil(index(2.0)) == 2


def test_plain_rotation_is_a_complex_multiplication_and_keeps_lengths():
    x = torch.randn(9, 3, 20, dtype=torch.float64)
    pos = torch.arange(40, 49)
    freqs, _ = plain.rotary_frequencies(12, 500.0)
    for interleaved in (True, False):
        y = plain.rotate(x, pos, freqs, 1.0, interleaved)
        assert torch.equal(y[..., 12:], x[..., 12:])            # the rest of a head passes unchanged
        a, b = (x[..., 0:12:2], x[..., 1:12:2]) if interleaved else (x[..., :6], x[..., 6:12])
        z = torch.complex(a, b) * torch.polar(torch.ones(9, 6, dtype=torch.float64),
                                              pos[:, None].double() * torch.tensor(freqs, dtype=torch.float64))[:, None, :]
        c, d = (y[..., 0:12:2], y[..., 1:12:2]) if interleaved else (y[..., :6], y[..., 6:12])
        torch.testing.assert_close(torch.complex(c, d), z)
    # scores of rotated vectors depend on the distance only
    q, k = torch.randn(1, 12, dtype=torch.float64), torch.randn(1, 12, dtype=torch.float64)
    s = [(plain.rotate(q, torch.tensor([p + 7]), freqs, 1.0, True) * plain.rotate(k, torch.tensor([p]), freqs, 1.0, True)).sum()
         for p in (0, 100, 1000)]
    assert s[0] == pytest.approx(s[1].item()) and s[0] == pytest.approx(s[2].item())


def test_plain_softmax_with_a_sink_and_the_visibility_rule():
    s = torch.randn(2, 6, 6, dtype=torch.float64)
    sink = torch.tensor([0.7, -30.0], dtype=torch.float64)
    mask = plain.visible(6)
    p = plain.softmax_rows(s, mask, sink)
    ref = torch.softmax(torch.cat([s.masked_fill(~mask, -math.inf), sink[:, None, None].expand(2, 6, 1)], dim=-1), dim=-1)
    torch.testing.assert_close(p, ref[..., :6])
    assert (p.sum(-1)[0] < 1).all() and torch.allclose(p.sum(-1)[1], torch.ones(6, dtype=torch.float64))
    vis = plain.visible(12, window=4, keep_first=2)
    assert vis[11].tolist() == [True, True] + [False] * 6 + [True] * 4
    assert vis[3].tolist() == [True] * 4 + [False] * 8
    assert plain.visible(5, window=0, keep_first=3).tolist() == torch.tril(torch.ones(5, 5)).bool().tolist()


def test_plain_layer_norm_and_latent_attention_against_library_routines():
    x, w = torch.randn(5, 40, dtype=torch.float64) * 3 + 2, torch.rand(40, dtype=torch.float64)
    torch.testing.assert_close(plain.layer_norm(x, w, 1e-5), torch.nn.functional.layer_norm(x, (40,), w, None, 1e-5))
    # latent attention with keys and values written out per head equals the same scores taken on
    # the latent rows with the key expansion moved to the query (the form the engine computes)
    cfg = U.CFG_R["layers"][0]["mixer"]
    H, d, r, dv, rank = cfg["heads"], cfg["dim"], cfg["rot_dim"], cfg["vdim"], cfg["kv_rank"]
    g = torch.Generator().manual_seed(0)
    wts = {"m.q": torch.randn(H * (d + r), 64, generator=g), "m.dkv": torch.randn(rank + r, 64, generator=g),
           "m.dkv.norm": torch.rand(rank, generator=g) + 0.5, "m.uk": torch.randn(H * d, rank, generator=g),
           "m.uv": torch.randn(H * dv, rank, generator=g), "m.sink": torch.randn(H, generator=g),
           "m.g": torch.randn(H, 64, generator=g), "m.o": torch.randn(64, H * dv, generator=g)}
    wts = {k: v.double() * 0.2 for k, v in wts.items()}
    h = torch.randn(11, 64, dtype=torch.float64, generator=g)
    want = plain.latent_attention(h, wts, "m.", cfg, 1e-6)
    pos = torch.arange(11)
    freqs, mag = plain.rotary_frequencies(r, cfg["rot"]["base"])
    q = (h @ wts["m.q"].T).view(11, H, d + r)
    down = h @ wts["m.dkv"].T
    c = plain.unit_rms(down[:, :rank], 1e-6) * wts["m.dkv.norm"]
    row = torch.cat([c, plain.rotate(down[:, rank:], pos, freqs, mag, False)], dim=-1)
    q_lat = torch.cat([torch.einsum("thd,hdr->thr", q[..., :d], wts["m.uk"].view(H, d, rank)),
                       plain.rotate(q[..., d:], pos, freqs, mag, False)], dim=-1)
    prob = plain.softmax_rows(torch.einsum("ihk,jk->hij", q_lat, row) * cfg["scale"], plain.visible(11), wts["m.sink"])
    o_lat = torch.einsum("hij,jr->ihr", prob, c)
    out = torch.einsum("ihr,hvr->ihv", o_lat, wts["m.uv"].view(H, dv, rank)) * torch.sigmoid(h @ wts["m.g"].T)[..., None]
    torch.testing.assert_close(out.reshape(11, H * dv) @ wts["m.o"].T, want)


def manager(window, keep_first, pages=12, page=4, seats=2):
    groups = [(attention_cache_spec(1, 8, kind="window", window=window, keep_first=keep_first), [0]),
              (latent_cache_spec(6, 2), [1])]
    return CacheManager(groups, {}, page_size=page, num_pages=pages, max_seqs=seats, max_seq_len=pages * page)


def test_a_window_group_keeps_the_pages_of_the_first_positions():
    cm = manager(window=6, keep_first=5)            # pages of 4: blocks 0 and 1 hold kept positions
    seat = cm.admit("a")
    win, full = cm.groups
    assert win.kept_blocks == 2
    for length in range(1, 41):
        assert cm.grow(seat, length)
        cm.slot_mapping(seat, length - 1, 1, 0)
        cm.commit(seat, length)
        cm.check()
        row = win.table_host[seat]
        first_needed = max(0, length - 6 + 1) // 4
        for b in range((length + 3) // 4):
            assert (row[b] >= 0) == (b < 2 or b >= first_needed), (length, b)
        assert (full.table_host[seat][:(length + 3) // 4] >= 0).all()
    held = win.num_pages - win.free_pages()
    assert held <= 2 + 3                             # the kept head and what a window of 6 touches
    cm.free(seat)
    cm.check()
    assert win.free_pages() == win.num_pages and full.free_pages() == full.num_pages
    # the pages come back to another request, the kept ones too
    seat = cm.admit("b")
    assert cm.grow(seat, 48)
    cm.commit(seat, 48)
    cm.check()
    assert win.pool.reuses > 0


def test_pages_a_window_group_needs_count_the_kept_ones():
    cm = manager(window=6, keep_first=5, pages=64)
    win, full = cm.groups
    assert full.pages_for(100) == 25
    assert win.pages_for(100, portion=8) == (6 - 1 + 8 + 3) // 4 + 1 + 2
    assert win.pages_for(7, portion=8) == 2          # never more than the prompt has
    no_keep = manager(window=6, keep_first=0).groups[0]
    assert no_keep.kept_blocks == 0 and no_keep.pages_for(100, portion=8) == (6 - 1 + 8 + 3) // 4 + 1
