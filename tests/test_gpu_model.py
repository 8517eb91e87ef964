"""End to end on a transformers decoder, the way the reference is used (tests/test_quantization.py:36-52 of
the reference: build a causal LM, Bitween(model, bits=4, group_size=64).quantize(rtn=True,
ignore_layers=[...]), run it, torch.save it).  The reference's test downloads facebook/opt-125m; there is no
network here, so the model is a randomly initialised Llama of the same kind of size.

The expected logits come from the same model with every quantised layer replaced by an fp16 nn.Linear that
holds W16 = fp16(scale * (q - zp)) computed by the ORACLE from the module's buffers - i.e. what the
reference's forward multiplies with (bitween/modules.py:85-101)."""
import copy
import io

import numpy as np
import pytest
import torch

from oracle import rtn_oracle as orc

pytestmark = pytest.mark.gpu

transformers = pytest.importorskip("transformers")


def _tiny_llama(seed=0):
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(seed)
    cfg = LlamaConfig(hidden_size=256, intermediate_size=768, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, vocab_size=512, max_position_embeddings=256, tie_word_embeddings=False)
    model = LlamaForCausalLM(cfg)
    # a random decoder's logits are nearly flat; make the weights large enough that the layers matter
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() == 2:
                p.mul_(4.0)
    return model.half().cuda().eval()


def _oracle_twin(qmodel):
    """qmodel with every QuantizedLinear turned back into an fp16 nn.Linear holding the oracle's W16."""
    import bitween_amd
    from bitween_amd.quantizer.func import _set_module
    twin = copy.deepcopy(qmodel)
    for name, mod in list(twin.named_modules()):
        if isinstance(mod, bitween_amd.QuantizedLinear):
            w16 = orc.dequantize_f16(mod.qweight.cpu().numpy(), mod.scale.cpu().numpy(), mod.zero_point.cpu().numpy(),
                                     mod.group_size, mod.bits)
            lin = torch.nn.Linear(mod.in_features, mod.out_features, bias=mod.bias is not None, device="cuda",
                                  dtype=torch.float16)
            lin.weight.data = torch.from_numpy(np.ascontiguousarray(w16)).cuda()
            if mod.bias is not None:
                lin.bias.data = mod.bias.data.clone()
            _set_module(twin, name, lin)
    return twin


@pytest.mark.parametrize("fuse", [False, True])
def test_llama_quantize_forward_generate_save(fuse):
    import bitween_amd
    model = _tiny_llama()
    n_linear = sum(isinstance(m, torch.nn.Linear) for m in model.modules())
    quantizer = bitween_amd.Bitween(model, tokenizer=None, bits=4, group_size=64)
    qmodel = quantizer.quantize(rtn=True, ignore_layers=["lm_head", "embed_tokens"], verbose=False, fuse_siblings=fuse)
    layers = [m for m in qmodel.modules() if isinstance(m, bitween_amd.QuantizedLinear)]
    assert len(layers) == n_linear - 1                        # everything but lm_head
    assert isinstance(qmodel.lm_head, torch.nn.Linear)
    assert all(isinstance(m, torch.nn.Linear) for m in model.modules() if hasattr(m, "in_features"))   # input untouched

    twin = _oracle_twin(qmodel)
    gen = torch.Generator(device="cuda").manual_seed(5)
    for shape in ((1, 1), (1, 7), (2, 33), (1, 130)):          # decode kernel, its 16-row slices, prefill kernel
        ids = torch.randint(0, 512, shape, device="cuda", generator=gen)
        with torch.no_grad():
            got = qmodel(input_ids=ids).logits.float()
            want = twin(input_ids=ids).logits.float()
        assert torch.isfinite(got).all()
        # every linear is within 1e-2 of the fp16 GEMM (main.py:471-477 of the reference); two layers deep the
        # logits stay within a few times that
        assert (got - want).abs().max().item() <= 3e-2 * want.abs().max().item()
        assert (got - want).abs().mean().item() <= 1e-2 * want.abs().mean().item()

    ids = torch.randint(0, 512, (1, 12), device="cuda", generator=gen)
    with torch.no_grad():
        out = qmodel.generate(ids, max_new_tokens=8, do_sample=False, use_cache=True, pad_token_id=0)
    assert out.shape == (1, 20) and torch.equal(out[:, :12], ids)
    # every greedy step picked a token whose logit in the twin is (all but) the twin's maximum
    with torch.no_grad():
        twin_logits = twin(input_ids=out[:, :-1]).logits.float()
    for t in range(12, 20):
        row = twin_logits[0, t - 1]
        assert row[out[0, t]].item() >= row.max().item() - 3e-2 * row.abs().max().item()

    # whole-module pickle, as the reference saves its models (main.py:134-145)
    buf = io.BytesIO()
    torch.save(qmodel, buf)
    buf.seek(0)
    loaded = torch.load(buf, weights_only=False)               # our own file, written two lines above
    with torch.no_grad():
        again = loaded(input_ids=ids).logits
        first = qmodel(input_ids=ids).logits
    assert torch.equal(again, first)


def test_llama_mixed_precision_map():
    """A per-block (bits, group) map on the same decoder: attention 8-bit g128, MLP 4-bit g128, one down_proj
    2-bit g32 - the shape of the mixed-precision benchmark configuration."""
    import bitween_amd
    model = _tiny_llama(seed=1)
    cfg = {"model.layers.0.self_attn": (8, 128), "model.layers.1.self_attn": (8, 128),
           "model.layers.0.mlp": (4, 128), "model.layers.1.mlp": (4, 128), "model.layers.1.mlp.down_proj": (2, 32)}
    qmodel = bitween_amd.Bitween(model, bits=4, group_size=128).quantize(
        rtn=True, ignore_layers=["lm_head"], layer_config=cfg, verbose=False)
    assert (qmodel.model.layers[1].mlp.down_proj.bits, qmodel.model.layers[1].mlp.down_proj.group_size) == (2, 32)
    assert qmodel.model.layers[0].self_attn.q_proj.bits == 8 and qmodel.model.layers[0].mlp.up_proj.bits == 4
    twin = _oracle_twin(qmodel)
    ids = torch.randint(0, 512, (1, 40), device="cuda", generator=torch.Generator(device="cuda").manual_seed(9))
    with torch.no_grad():
        got = qmodel(input_ids=ids).logits.float()
        want = twin(input_ids=ids).logits.float()
    assert (got - want).abs().max().item() <= 3e-2 * want.abs().max().item()


def test_decoder_step_under_graph_capture_equals_the_eager_step():
    """bench_decoder.Decoder (the end-to-end configuration of bench.py) on a 2-layer model with the mixed recipe:
    a decode step captured in a HIP graph and replayed gives the logits and the tokens of the eager step, token
    after token; and the quantised model agrees with a float16 twin built from the oracle's W16."""
    import bench_decoder as bd
    from bitween_amd import Bitween, QuantizedLinear
    torch.manual_seed(0)
    with torch.device("cuda"):
        model = bd.Decoder(layers=2, hidden=256, heads=4, inter=512, vocab=1000, max_len=96).half()
    model.init_weights(seed=3)
    recipe = {"layers.0.self_attn": (8, 128), "layers.1.self_attn": (8, 128), "layers.0.mlp": (4, 128),
              "layers.1.mlp": (4, 128), "layers.1.mlp.down_proj": (2, 32)}
    q = Bitween(model, bits=4, group_size=128).quantize(rtn=True, ignore_layers=["lm_head", "embed_tokens"],
                                                        layer_config=recipe, verbose=False)
    kinds = {name: (m.bits, m.group_size) for name, m in q.named_modules() if isinstance(m, QuantizedLinear)}
    assert len(kinds) == 14 and kinds["layers.1.mlp.down_proj"] == (2, 32) and kinds["layers.0.self_attn.k_proj"] == (8, 128)
    assert isinstance(q.lm_head, torch.nn.Linear)
    q.alloc_state()
    ids = torch.randint(0, 1000, (40,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    _, _, toks_eager = bd.generate(q, ids, 24)
    # logits of the first decode step, eagerly
    q.prefill(ids)
    logits_eager = q.step().clone()
    graph = bd.capture_step(q)
    q.prefill(ids)
    # capture ran one warm-up step: find the captured step's output tensor by replaying
    graph.replay()
    torch.cuda.synchronize()
    assert int(q.pos) == 41
    assert torch.equal(q.out[40:41], toks_eager[1:2])
    _, _, toks_graph = bd.generate(q, ids, 24, graph)
    assert torch.equal(toks_graph, toks_eager)
    # the float16 twin: same decoder, every quantised linear replaced by nn.Linear holding W16
    from bitween_amd.kernels import hip_loader as hip
    twin = copy.deepcopy(q)
    for name, m in list(twin.named_modules()):
        if isinstance(m, QuantizedLinear):
            lin = torch.nn.Linear(m.in_features, m.out_features, bias=False, device="cuda", dtype=torch.float16)
            lin.weight.data = hip.dequantize(m.qweight, m.scale, m.zero_point, m.group_size, m.bits, torch.float16)
            parent = twin
            *path, leaf = name.split(".")
            for part in path:
                parent = getattr(parent, part)
            setattr(parent, leaf, lin)
    twin.alloc_state()
    twin.prefill(ids)
    logits_twin = twin.step()
    rel = (logits_eager.float() - logits_twin.float()).abs().max() / logits_twin.float().abs().max()
    assert rel < 2e-2


def test_full_size_decoder_layer_with_the_mixed_recipe_against_the_oracle():
    """The end-to-end configuration at its real widths: one decoder layer of bench_decoder.Decoder with hidden 4096,
    32 heads, MLP 11008, vocab 32000 and the mixed recipe (attention 8-bit g128, gate / up 4-bit g128, down_proj 2-bit
    g32), quantised by Bitween(...).quantize.  Every quantised linear is checked against the oracle on sampled rows
    (packed words, float16 scales and zero points, W16 bit for bit); the logits of the first decode step - one launch
    per module, then with q/k/v and gate/up sharing launches - are compared with a float16 twin that holds W16."""
    import bench_decoder as bd
    import bitween_amd
    from bitween_amd import Bitween, QuantizedLinear
    from bitween_amd.kernels import hip_loader as hip
    with torch.device("cuda"):
        model = bd.Decoder(layers=1, hidden=4096, heads=32, inter=11008, vocab=32000, max_len=64).half()
    model.init_weights(seed=5)
    recipe = {"layers.0.self_attn": (8, 128), "layers.0.mlp": (4, 128), "layers.0.mlp.down_proj": (2, 32)}
    originals = {name: m.weight.data for name, m in model.named_modules() if isinstance(m, torch.nn.Linear)}
    q = Bitween(model, bits=4, group_size=128).quantize(rtn=True, ignore_layers=["lm_head", "embed_tokens"],
                                                        layer_config=recipe, verbose=False)
    qlin = {name: m for name, m in q.named_modules() if isinstance(m, QuantizedLinear)}
    assert sorted((m.bits, m.group_size) for m in qlin.values()) == [(2, 32)] + [(4, 128)] * 2 + [(8, 128)] * 4
    twin = copy.deepcopy(q)
    for name, m in qlin.items():
        w16 = hip.dequantize(m.qweight, m.scale, m.zero_point, m.group_size, m.bits, torch.float16)
        rows = np.unique(np.concatenate([np.arange(0, m.out_features, m.out_features // 16), [m.out_features - 1]]))
        w_rows = originals[name][rows].float().cpu().numpy()
        qw_o, s_o, z_o, _ = orc.quantize_rtn(w_rows, m.bits, m.group_size)
        s16, z16 = orc.store_module_buffers(s_o, z_o)
        assert np.array_equal(m.qweight[rows].cpu().numpy(), qw_o), name
        assert np.array_equal(m.scale[rows].cpu().numpy().view(np.uint16), s16.view(np.uint16)), name
        assert np.array_equal(m.zero_point[rows].cpu().numpy(), z16), name
        w16_o = orc.dequantize_f16(qw_o, s16, z16, m.group_size, m.bits)
        assert np.array_equal(w16[rows].cpu().numpy().view(np.uint16), w16_o.view(np.uint16)), name
        lin = torch.nn.Linear(m.in_features, m.out_features, bias=False, device="cuda", dtype=torch.float16)
        lin.weight.data = w16
        parent = twin
        *path, leaf = name.split(".")
        for part in path:
            parent = getattr(parent, part)
        setattr(parent, leaf, lin)
    ids = torch.randint(0, 32000, (24,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    twin.alloc_state()
    twin.prefill(ids)
    want = twin.step().float()
    q.alloc_state()
    q.prefill(ids)
    got = q.step().float()
    assert (got - want).abs().max().item() <= 2e-2 * want.abs().max().item()
    assert bitween_amd.fuse_sibling_linears(q) == 2
    q.prefill(ids)
    fused = q.step().float()
    assert (fused - want).abs().max().item() <= 2e-2 * want.abs().max().item()
    # the fused launches run the same arithmetic over concatenated rows (another split of K over waves at most)
    assert (fused - got).abs().max().item() <= 2e-3 * want.abs().max().item()
