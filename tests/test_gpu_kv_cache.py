"""The preallocated prefix cache against the reference's flow (slice, cat, repeat) run on the oracle."""

import pytest
import torch

from opentau_amd import flash_attn_hip as fa
from opentau_amd.kv_cache import StaticKVCache
from opentau_amd.rope import apply_rope_qk, rope_raw
from oracle import eager
from oracle import rope as oracle_rope
from tests.helpers import assert_close_bf16, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def g(t):
    return t.to(DEV)


@pytest.mark.parametrize("n_cand", [1, 4])
def test_denoise_flow_through_the_static_cache(n_cand):
    """pi0.5 inference in small: a prefix pass fills the cache layer by layer (keys rotated straight into
    it), then denoise steps attend [cache ; own K/V]; with n_cand > 1 the candidates share the cache.
    The oracle runs the reference's flow: apply_rope, slice into past_key_values, repeat for the
    candidates, concatenate per layer and step, eager attention with the dense mask."""
    layers, b, n_pre, n_act, h, hkv, d, steps = 3, 2, 140, 50, 8, 1, 256, 2
    dt = torch.bfloat16
    pre_pad = torch.ones(b, n_pre, dtype=torch.bool)
    pre_pad[0, -9:] = False
    pre_att = torch.zeros(b, n_pre, dtype=torch.int32)
    pre_pos = (torch.cumsum(pre_pad, 1) - 1).clamp_min(0)
    cache = StaticKVCache(layers, b, 256, hkv, d, dt, DEV)
    pre_ids = [g(t) for t in fa.make_att_block_ids(pre_pad, pre_att)]
    ref_past = {}
    for layer in range(layers):
        q, k, v = (randn((b, n_pre, hh, d), dt, 10 * layer + i) for i, hh in enumerate((h, hkv, hkv)))
        # product: q rotated in place, k rotated into the cache rows, v copied there
        qg = g(q)
        rope_raw(qg, None, g(pre_pos), q_out=qg)
        k_rows, v_rows = cache.fill(layer, g(k), g(v), positions=g(pre_pos))
        out = fa.flash_attn_blockmask(qg, k_rows, v_rows, *pre_ids, d**-0.5)
        # oracle
        q_r, k_r = oracle_rope.apply_rope(q, pre_pos), oracle_rope.apply_rope(k, pre_pos)
        ref_past[layer] = {"key_states": k_r, "value_states": v}
        ref = eager.eager_from_block_ids(q_r, k_r, v, *fa.make_att_block_ids(pre_pad, pre_att), d**-0.5)
        valid = pre_pad[:, :, None, None]
        assert_close_bf16((out.cpu() * valid).float(), (ref * valid).float(), f"prefix layer {layer}")
    assert cache.length == n_pre
    past = cache.as_past_key_values()
    assert sorted(past) == list(range(layers)) and past[1]["key_states"].shape == (b, n_pre, hkv, d)

    # denoise steps: B * n_cand candidates in (b n) order
    bn = b * n_cand
    suf_pad = torch.ones(bn, n_act, dtype=torch.bool)
    suf_att = torch.zeros(bn, n_act, dtype=torch.int32)
    suf_att[:, 0] = 1
    cross_pad = pre_pad.repeat_interleave(n_cand, 0)
    ids_cpu = fa.make_att_block_ids(suf_pad, suf_att, n_pre, cross_pad)
    ids = tuple(g(t) for t in ids_cpu)
    suf_pos = cross_pad.sum(1, keepdim=True) + torch.arange(n_act)[None]
    for step in range(steps):
        for layer in range(layers):
            q, k, v = (randn((bn, n_act, hh, d), dt, 1000 + 100 * step + 10 * layer + i)
                       for i, hh in enumerate((h, hkv, hkv)))
            qg, kg = apply_rope_qk(g(q), g(k), g(suf_pos))
            out = cache.attend(layer, qg, kg, g(v), ids)
            assert out.shape == (bn, n_act, h * d)
            kc = ref_past[layer]["key_states"].repeat_interleave(n_cand, 0)
            vc = ref_past[layer]["value_states"].repeat_interleave(n_cand, 0)
            k_all = torch.cat([kc, oracle_rope.apply_rope(k, suf_pos)], 1)
            v_all = torch.cat([vc, v], 1)
            ref = eager.eager_from_block_ids(oracle_rope.apply_rope(q, suf_pos), k_all, v_all, *ids_cpu, d**-0.5)
            assert_close_bf16(out.reshape(bn, n_act, h, d).float().cpu(), ref.float(), f"step {step} layer {layer}")
    # the summary was computed once: a fresh call without the shared workspace gives the same bits
    kc, vc = cache.layer(layers - 1)
    again, _ = fa.forward_raw(qg, kc, vc, *ids, d**-0.5, kg, g(v), kvcache=True)
    assert torch.equal(again.reshape(out.shape), out)


def test_cache_rejects_rows_that_do_not_fit():
    cache = StaticKVCache(1, 2, 16, 1, 64, torch.bfloat16, DEV)
    k = g(randn((2, 17, 1, 64), torch.bfloat16, 1))
    with pytest.raises(RuntimeError, match="fit"):
        cache.fill(0, k, k)
    with pytest.raises(RuntimeError, match="fit"):
        cache.fill(0, k[:1, :4], k[:1, :4])


def test_whole_denoise_loop_replays_from_one_graph():
    """The pi0.5 inference loop at its real depth, 10 flow-matching steps x 18 layers of [rotate q and k ;
    attend over the cached prefix and the step's own keys] through the static cache
    (``pi05/modeling_pi05.py:2015-2046``, ``paligemma_with_expert.py:742-768``), captured as ONE HIP graph:
    every replay, on new inputs in the captured buffers and with eager work in between, gives bit for bit
    what the same loop gives when called eagerly (the mask's summary is made once, before the capture; the
    calls allocate through the graph's pool only and clear nothing)."""
    layers, steps, b, n_pre, n_act, h, hkv, d = 18, 10, 2, 200, 50, 8, 1, 256
    dt = torch.bfloat16
    pre_pad = torch.ones(b, n_pre, dtype=torch.bool)
    pre_pad[1, -13:] = False
    pre_pos = (torch.cumsum(pre_pad, 1) - 1).clamp_min(0)
    cache = StaticKVCache(layers, b, 256, hkv, d, dt, DEV)
    for layer in range(layers):
        cache.fill(layer, g(randn((b, n_pre, hkv, d), dt, 3 * layer)), g(randn((b, n_pre, hkv, d), dt, 3 * layer + 1)),
                   positions=g(pre_pos))
    suf_pad = torch.ones(b, n_act, dtype=torch.bool)
    suf_att = torch.zeros(b, n_act, dtype=torch.int32)
    suf_att[:, 0] = 1
    ids = tuple(g(t) for t in fa.make_att_block_ids(suf_pad, suf_att, n_pre, pre_pad))
    suf_pos = g(pre_pad.sum(1, keepdim=True) + torch.arange(n_act)[None])
    qs = g(randn((layers, b, n_act, h, d), dt, 500))
    ks, vs = g(randn((layers, b, n_act, hkv, d), dt, 501)), g(randn((layers, b, n_act, hkv, d), dt, 502))

    def loop():
        outs = []
        for step in range(steps):
            gain = 1.0 + 0.03 * step  # (a step's inputs differ from the last step's)
            for layer in range(layers):
                q, k = apply_rope_qk(qs[layer] * gain, ks[layer], suf_pos)
                outs.append(cache.attend(layer, q, k, vs[layer], ids))
        return outs

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):  # first calls outside the capture: kernel attributes, the mask's summary
        loop()
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = loop()
    assert len(captured) == steps * layers
    for rep in range(3):
        for t, seed in ((qs, 600), (ks, 601), (vs, 602)):
            t.copy_(g(randn(tuple(t.shape), dt, seed + 10 * rep)))
        graph.replay()
        torch.cuda.synchronize()
        eager_outs = loop()
        torch.cuda.synchronize()
        assert all(torch.equal(a, e) for a, e in zip(captured, eager_outs)), rep
        assert float(captured[-1].float().abs().sum()) > 0
