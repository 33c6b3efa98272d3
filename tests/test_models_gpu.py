"""Whole models on the drop-in path: small random-init ``transformers`` models with
``attn_implementation="sdpa"`` run one training step (loss and every parameter gradient) and a greedy
generation with the stock attention kernels of this PyTorch build and again with this package
registered.  The models reach the operators the way real callers do: ``is_causal`` without a mask,
additive padding + causal masks built by the model code, sliding-window masks, grouped heads with
``enable_gqa``, head dim 256, bidirectional padding masks, 197-token images.  Not a parity test against
the oracle (those are the kernel and operator tests): it checks that nothing between the model code and
the kernels - mask recognition, layouts, autograd, the KV-cache decode steps - changes the numbers.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu

transformers = pytest.importorskip("transformers")


@pytest.fixture(scope="module")
def amd(gpu_device):
    import torch_neuronx_amd as amd

    return amd


def _llama(**kw):
    cfg = dict(vocab_size=1000, hidden_size=512, intermediate_size=1024, num_hidden_layers=2,
               num_attention_heads=8, num_key_value_heads=2, attn_implementation="sdpa")
    cfg.update(kw)
    return transformers.LlamaForCausalLM(transformers.LlamaConfig(**cfg))


def _mistral():
    return transformers.MistralForCausalLM(transformers.MistralConfig(
        vocab_size=1000, hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8,
        num_key_value_heads=2, sliding_window=64, attn_implementation="sdpa"))


def _gemma2():
    return transformers.Gemma2ForCausalLM(transformers.Gemma2Config(
        vocab_size=1000, hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, head_dim=256, sliding_window=64, attn_implementation="sdpa"))


def _gpt2():
    return transformers.GPT2LMHeadModel(transformers.GPT2Config(
        vocab_size=1000, n_embd=384, n_layer=2, n_head=6, n_positions=512, attn_pdrop=0.0, resid_pdrop=0.0,
        embd_pdrop=0.0, bos_token_id=0, eos_token_id=0, attn_implementation="sdpa"))


def _bert():
    return transformers.BertForMaskedLM(transformers.BertConfig(
        vocab_size=1000, hidden_size=384, num_hidden_layers=2, num_attention_heads=6, intermediate_size=768,
        hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, attn_implementation="sdpa"))


def _vit():
    return transformers.ViTModel(transformers.ViTConfig(
        hidden_size=384, num_hidden_layers=2, num_attention_heads=6, intermediate_size=768,
        hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0, attn_implementation="sdpa"))


CASES = {
    "llama_gqa_no_mask": (_llama, False, torch.bfloat16),
    "llama_gqa_padding": (_llama, True, torch.bfloat16),
    "llama_gqa_padding_float32": (_llama, True, torch.float32),
    "mistral_sliding_window": (_mistral, True, torch.bfloat16),
    "gemma2_head_dim_256": (_gemma2, True, torch.bfloat16),
    "gpt2_float32": (_gpt2, True, torch.float32),
    "bert_padding": (_bert, True, torch.bfloat16),
    "bert_padding_float32": (_bert, True, torch.float32),
    "vit_197_tokens": (_vit, None, torch.bfloat16),
}


def _step(model, inputs):
    model.zero_grad()
    out = model(**inputs)
    loss = out.loss if getattr(out, "loss", None) is not None else out[0].float().square().mean()
    loss.backward()
    return loss.detach().float(), torch.cat([p.grad.float().flatten() for p in model.parameters() if p.grad is not None])


@pytest.fixture
def library_calls(amd, monkeypatch):
    seen = {"fwd": 0, "bwd": 0}
    f0, b0 = amd.ops.sdpa_forward, amd.ops.sdpa_backward

    def f(*a, **k):
        seen["fwd"] += 1
        return f0(*a, **k)

    def b(*a, **k):
        seen["bwd"] += 1
        return b0(*a, **k)

    monkeypatch.setattr(amd.ops, "sdpa_forward", f)
    monkeypatch.setattr(amd.ops, "sdpa_backward", b)
    return seen


@pytest.mark.parametrize("name", list(CASES))
def test_training_step_of_a_model_matches_the_stock_kernels(amd, gpu_device, library_calls, name):
    make, padded, dtype = CASES[name]
    dev = gpu_device
    torch.manual_seed(1)
    model = make().to(dev).to(dtype).train()
    B, S = 4, 256
    if padded is None:
        inputs = dict(pixel_values=torch.randn(B, 3, 224, 224, device=dev, dtype=dtype))
    else:
        ids = torch.randint(1, 1000, (B, S), device=dev)
        inputs = dict(input_ids=ids, labels=ids)
        if padded:
            am = torch.ones(B, S, dtype=torch.long, device=dev)
            am[1, 200:] = 0
            am[3, 100:] = 0
            inputs["attention_mask"] = am
    try:
        amd.unregister()
        l0, g0 = _step(model, inputs)
        assert library_calls == {"fwd": 0, "bwd": 0}
    finally:
        amd.register()
    l1, g1 = _step(model, inputs)
    assert library_calls["fwd"] == 2 and library_calls["bwd"] == 2, library_calls  # (one call per layer)
    rel = float((g1 - g0).norm() / g0.norm())
    if dtype is torch.float32:
        assert abs(float(l1 - l0)) <= 1e-5 and rel <= 1e-5, (float(l0), float(l1), rel)
    else:  # two bf16 implementations: each rounds the output and the gradients once per layer
        assert abs(float(l1 - l0)) <= 2e-3 and rel <= 2e-2, (float(l0), float(l1), rel)


@pytest.mark.parametrize("left_padding", [False, True])
def test_greedy_generation_with_a_kv_cache_matches_the_stock_kernels(amd, gpu_device, library_calls, left_padding):
    """Prefill, then 24 decode steps of one query row against the growing cache; float32 with grouped
    heads, which upstream's backend choice sends to its unfused path - routed to the library by
    ``route_functional``, the reference's backend choice.  The tokens are the stock ones."""
    dev = gpu_device
    torch.manual_seed(1)
    model = _llama().to(dev).eval()
    ids = torch.randint(1, 1000, (4, 32), device=dev)
    am = torch.ones_like(ids)
    if left_padding:
        am[1, :7] = 0
        am[2, :20] = 0
    try:
        amd.unregister()
        with torch.no_grad():
            want = model.generate(ids, attention_mask=am, max_new_tokens=24, do_sample=False)
    finally:
        amd.register()
    amd.route_functional(True)
    try:
        with torch.no_grad():
            got = model.generate(ids, attention_mask=am, max_new_tokens=24, do_sample=False)
    finally:
        amd.route_functional(False)
    assert library_calls["fwd"] == 48, library_calls
    assert torch.equal(got, want)


@pytest.mark.parametrize("case", ["no_mask", "key_padding", "causal_flag", "causal_and_padding", "eval_fast_path",
                                  "encoder_padding", "decoder_layer"])
def test_torch_nn_attention_modules_match_the_stock_kernels(amd, gpu_device, library_calls, case):
    """``nn.MultiheadAttention`` / ``nn.TransformerEncoder`` / ``nn.TransformerDecoderLayer`` in float32:
    the masks these modules merge (key padding expanded per head, a causal mask with the flag, both) and
    the inference fast path reach the library and give the stock numbers, outputs and gradients."""
    import torch.nn as nn

    dev = gpu_device
    B, S, E, H = 8, 200, 384, 6
    torch.manual_seed(0)
    x = torch.randn(B, S, E, device=dev)
    pad = torch.zeros(B, S, dtype=torch.bool, device=dev)
    pad[1, 150:] = True
    pad[5, 60:] = True
    causal = nn.Transformer.generate_square_subsequent_mask(S, device=dev)
    if case == "encoder_padding":
        mod, args, kw, calls = nn.TransformerEncoder(nn.TransformerEncoderLayer(E, H, 768, dropout=0.0, batch_first=True), 2), (x,), dict(src_key_padding_mask=pad), 2
    elif case == "decoder_layer":
        mod, args, calls = nn.TransformerDecoderLayer(E, H, 768, dropout=0.0, batch_first=True), (x, x), 2
        kw = dict(tgt_mask=causal, tgt_is_causal=True, memory_key_padding_mask=pad)
    else:
        mod, args, calls = nn.MultiheadAttention(E, H, batch_first=True, dropout=0.0), (x, x, x), 1
        kw = {"no_mask": {}, "eval_fast_path": {}, "key_padding": dict(key_padding_mask=pad),
              "causal_flag": dict(attn_mask=causal, is_causal=True),
              "causal_and_padding": dict(attn_mask=causal, key_padding_mask=pad.float().masked_fill(pad, float("-inf")))}[case]
        kw["need_weights"] = False
    mod = mod.to(dev)
    train = case != "eval_fast_path"

    def run():
        mod.train(train)
        mod.zero_grad()
        with torch.set_grad_enabled(train):
            out = mod(*args, **kw)
            out = out[0] if isinstance(out, tuple) else out
            if train:
                out.square().mean().backward()
        return out.detach(), (torch.cat([p.grad.flatten() for p in mod.parameters()]) if train else None)

    try:
        amd.unregister()
        o0, g0 = run()
        assert library_calls == {"fwd": 0, "bwd": 0}
    finally:
        amd.register()
    o1, g1 = run()
    assert library_calls["fwd"] == calls and library_calls["bwd"] == (calls if train else 0), library_calls
    assert float((o1 - o0).abs().max()) <= 1e-5 * max(1.0, float(o0.abs().max()))
    if train:
        assert float((g1 - g0).norm() / g0.norm()) <= 1e-5


def test_a_compiled_model_reaches_the_library_and_matches_eager(amd, gpu_device, library_calls):
    """A whole model under ``torch.compile`` (default backend), float32, padded batch: the generated code
    calls the registered operators - it asserts their output shapes and strides on the way - once per layer
    and direction, and loss and gradients are the eager ones."""
    dev = gpu_device
    torch.manual_seed(1)
    model = _llama().to(dev).train()
    ids = torch.randint(1, 1000, (4, 256), device=dev)
    am = torch.ones_like(ids)
    am[1, 200:] = 0
    am[3, 100:] = 0
    inputs = dict(input_ids=ids, labels=ids, attention_mask=am)
    l0, g0 = _step(model, inputs)
    before = dict(library_calls)
    torch._dynamo.reset()
    try:
        l1, g1 = _step(torch.compile(model), inputs)
    finally:
        torch._dynamo.reset()
    assert library_calls["fwd"] - before["fwd"] == 2 and library_calls["bwd"] - before["bwd"] == 2, library_calls
    assert abs(float(l1 - l0)) <= 1e-5 and float((g1 - g0).norm() / g0.norm()) <= 1e-5
