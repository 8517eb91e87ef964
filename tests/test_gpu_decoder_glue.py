"""The glue kernels of the end-to-end decoder benchmark (bench_decoder_glue.hip) against the torch operations they
stand for, at the benchmark's sizes (hidden 4096, 32 heads of 128, 768 cached positions), and the decoder's decode
step through them against the same step through torch's ops.  float32 arithmetic with one rounding to float16
against torch's per-operation float16 roundings: the bars below are a few float16 ulps of the largest value."""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu

bd = pytest.importorskip("bench_decoder")


@pytest.fixture(scope="module")
def small():
    if not os.path.exists(bd.GLUE_LIB):
        pytest.fail(f"{bd.GLUE_LIB} is not built (run __graft_entry__.build() on the CPU box first)")
    with torch.device("cuda"):
        model = bd.Decoder(layers=1, hidden=4096, heads=32, inter=11008, vocab=64, max_len=768).half()
    model.init_weights(seed=1)
    model.alloc_state()
    model.use_hip_glue(splits=8)
    return model


def rel(a, b):
    return ((a.float() - b.float()).abs().max() / b.float().abs().max().clamp_min(1e-6)).item()


def test_add_rmsnorm(small):
    g = small.glue
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(1, 4096, device="cuda", generator=gen).half()
    d = torch.randn(1, 4096, device="cuda", generator=gen).half()
    gamma = (1 + 0.1 * torch.randn(4096, device="cuda", generator=gen)).half()
    for delta in (d, None):
        x_out, h = g.add_rmsnorm(x, delta, gamma)
        want_x = x if delta is None else x + delta
        assert torch.equal(x_out, want_x)
        want_h = torch.nn.functional.rms_norm(want_x, (4096,), gamma, small.eps)
        assert rel(h, want_h) < 2e-3


@pytest.mark.parametrize("pos", [0, 1, 95, 96, 500, 767])
def test_rope_cache_write_and_attention(small, pos):
    m = small
    gen = torch.Generator(device="cuda").manual_seed(pos)
    m.kv.copy_(torch.randn(m.kv.shape, device="cuda", generator=gen).half())
    kv_before = m.kv.clone()
    m.pos.fill_(pos)
    q = torch.randn(1, 4096, device="cuda", generator=gen).half()
    k = torch.randn(1, 4096, device="cuda", generator=gen).half()
    v = torch.randn(1, 4096, device="cuda", generator=gen).half()
    q_rot = m.glue.rope_kv(q, k, v, 0)
    # torch: the decoder's own rotary code on q and k together
    m._cos, m._sin = m.cos.index_select(0, m.pos)[:, None, :], m.sin.index_select(0, m.pos)[:, None, :]
    qk = m._rope(torch.cat([q, k], dim=-1).view(1, 64, 128))
    assert rel(q_rot.view(32, 128), qk[0, :32]) < 2e-3
    assert rel(m.kv[0, 0, 0, :, pos], qk[0, 32:]) < 2e-3
    assert torch.equal(m.kv[0, 1, 0, :, pos], v.view(32, 128))
    # nothing but row `pos` of the two caches changed
    keep = torch.ones(768, dtype=torch.bool, device="cuda")
    keep[pos] = False
    assert torch.equal(m.kv[0][:, :, :, keep], kv_before[0][:, :, :, keep])
    # attention of the rotated query over positions 0 .. pos
    o = m.glue.attention(q_rot, 0)
    kc, vc = m.kv[0, 0, 0, :, : pos + 1].float(), m.kv[0, 1, 0, :, : pos + 1].float()       # [heads, n, 128]
    scores = torch.einsum("hd,hnd->hn", q_rot.view(32, 128).float(), kc) * 128 ** -0.5
    want = torch.einsum("hn,hnd->hd", torch.softmax(scores, dim=-1), vc)
    assert rel(o.view(32, 128), want) < 2e-3
    # the same in one call: rotary, cache write and attention (from the caches as they were before)
    kv_split = m.kv.clone()
    m.kv.copy_(kv_before)
    o_fused = m.glue.rope_attention(q, k, v, 0)
    assert torch.equal(m.kv, kv_split)
    assert rel(o_fused, o) < 1e-3


def test_silu_mul(small):
    gen = torch.Generator(device="cuda").manual_seed(5)
    gate = (3 * torch.randn(1, 11008, device="cuda", generator=gen)).half()
    up = torch.randn(1, 11008, device="cuda", generator=gen).half()
    got = small.glue.silu_mul(gate, up)
    want = torch.nn.functional.silu(gate) * up
    assert rel(got, want) < 2e-3


def test_entry_points_refuse_what_the_kernels_do_not_take(small):
    g = small.glue
    x = torch.zeros(1, 4096, device="cuda", dtype=torch.float16)
    null = None
    assert g.lib.glue_add_rmsnorm(x.data_ptr(), null, x.data_ptr(), x.data_ptr(), x.data_ptr(), 4100, 1e-5, null) == -1
    assert g.lib.glue_add_rmsnorm(x.data_ptr(), null, x.data_ptr(), x.data_ptr(), x.data_ptr(), 16384, 1e-5, null) == -1
    assert g.lib.glue_silu_mul(x.data_ptr(), x.data_ptr(), x.data_ptr(), 4, null) == -1
    # head dimension other than 128, slices longer than 256 positions
    args = [x.data_ptr()] * 6
    assert g.lib.glue_attention(*args, 32, 64, 768, 8, 1.0, null) == -1
    assert g.lib.glue_attention(*args, 32, 128, 768, 2, 1.0, null) == -1


def test_decode_step_through_hip_glue_matches_torch_glue_and_replays_under_a_graph():
    from bitween_amd import Bitween
    with torch.device("cuda"):
        model = bd.Decoder(layers=2, hidden=512, heads=4, inter=1024, vocab=1000, max_len=96).half()
    model.init_weights(seed=3)
    recipe = {"layers.0.self_attn": (8, 128), "layers.1.self_attn": (8, 128), "layers.0.mlp": (4, 128),
              "layers.1.mlp": (4, 128), "layers.1.mlp.down_proj": (2, 32)}
    q = Bitween(model, bits=4, group_size=128).quantize(rtn=True, ignore_layers=["lm_head", "embed_tokens"],
                                                        layer_config=recipe, verbose=False)
    q.alloc_state()
    ids = torch.randint(0, 1000, (40,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    q.prefill(ids)
    logits_torch = q.step().clone()
    kv_torch = q.kv.clone()
    q.use_hip_glue(splits=4)
    q.prefill(ids)
    logits_hip = q.step().clone()
    assert rel(logits_hip, logits_torch) < 1e-2
    assert rel(q.kv[:, :, :, :, :41], kv_torch[:, :, :, :, :41]) < 1e-2
    _, _, toks_eager = bd.generate(q, ids, 24)
    graph = bd.capture_step(q)
    _, _, toks_graph = bd.generate(q, ids, 24, graph)
    assert torch.equal(toks_graph, toks_eager)
    _, _, toks_again = bd.generate(q, ids, 24, graph)
    assert torch.equal(toks_again, toks_eager)
