"""Model code of the `transformers` library under the graph rewrite: tiny random-weight decoders and an encoder, their
attention written the library's own ways (the eager implementation with `repeat_kv`, additive masks, fp32 softmax and a
`.type()` / `.to()` cast back, Gemma 2's tanh soft-cap and sliding window; or calls of scaled_dot_product_attention).
Every layer's attention must become one fused launch, and the logits must be as close to the same model in fp32 on the
CPU as eager bf16 on the GPU is."""
import copy

import pytest
import torch

from flashlight_amd import fusion, ops

transformers = pytest.importorskip("transformers")

CONFIGS = {
    "llama": ("LlamaConfig", dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=8,
                                  num_key_value_heads=2, vocab_size=1000), True),
    "gpt2": ("GPT2Config", dict(n_embd=256, n_layer=2, n_head=4, vocab_size=1000, n_positions=256, bos_token_id=0,
                                eos_token_id=0), True),
    "bert": ("BertConfig", dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                                vocab_size=1000), False),
    "gemma2": ("Gemma2Config", dict(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                                    num_key_value_heads=2, head_dim=64, vocab_size=1000, sliding_window=64), True),
    "gptj": ("GPTJConfig", dict(n_embd=256, n_layer=2, n_head=4, rotary_dim=32, vocab_size=1000), True),          # fp32 q k^T
    "gpt_neo": ("GPTNeoConfig", dict(hidden_size=256, num_layers=2, num_heads=4, attention_types=[[["global", "local"], 1]],
                                     window_size=16, vocab_size=1000), True),
    "falcon": ("FalconConfig", dict(hidden_size=256, num_hidden_layers=2, num_attention_heads=4, vocab_size=1000), True),  # one K/V head
    "mpt": ("MptConfig", dict(d_model=256, n_layers=2, n_heads=4, vocab_size=1000), True),                         # ALiBi as a bias
}
CASES = [("llama", "eager", "flashlight_amd"), ("llama", "sdpa", "flashlight_amd"), ("llama", "eager", "flashlight_amd_inductor"),
         ("gpt2", "eager", "flashlight_amd"), ("bert", "eager", "flashlight_amd"), ("bert", "sdpa", "flashlight_amd"),
         ("gemma2", "eager", "flashlight_amd"), ("gemma2", "sdpa", "flashlight_amd_inductor"),
         ("gptj", "eager", "flashlight_amd"), ("gpt_neo", "eager", "flashlight_amd"), ("falcon", "sdpa", "flashlight_amd"),
         ("falcon", "eager", "flashlight_amd"), ("mpt", "eager", "flashlight_amd")]


@pytest.mark.gpu
@pytest.mark.parametrize("name,impl,backend", CASES)
def test_transformers_model(name, impl, backend):
    cls, kw, causal_lm = CONFIGS[name]
    if not hasattr(transformers, cls):
        pytest.skip(f"this transformers has no {cls}")
    torch.manual_seed(1)
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 1000, (2, 200), generator=g)
    attend = torch.ones(2, 200, dtype=torch.long)
    attend[1, :37] = 0   # left padding
    auto = transformers.AutoModelForCausalLM if causal_lm else transformers.AutoModel
    model = auto.from_config(getattr(transformers, cls)(**kw), attn_implementation=impl).eval()
    ref = copy.deepcopy(model).float()
    m = model.to(torch.bfloat16).to("cuda")
    first = lambda o: o.logits if hasattr(o, "logits") else o.last_hidden_state
    launches = [0]
    real = ops.dispatch

    def counting(*a, **k):
        launches[0] += 1
        return real(*a, **k)

    with torch.no_grad():
        want = first(ref(input_ids=ids, attention_mask=attend))
        eager = first(m(input_ids=ids.cuda(), attention_mask=attend.cuda())).float().cpu()
        torch._dynamo.reset()
        ops.dispatch = counting
        try:
            got = first(torch.compile(m, backend=backend, dynamic=False)(input_ids=ids.cuda(), attention_mask=attend.cuda()))
        finally:
            ops.dispatch = real
    got = got.float().cpu()
    keep = attend.bool()   # what a model computes at padded positions is arbitrary
    assert launches[0] >= 2, "both layers' attention on the fused kernel"
    if backend == "flashlight_amd":
        assert launches[0] == 2
    assert torch.isfinite(got[keep]).all()
    err, yard = (got - want)[keep].abs().max().item(), (eager - want)[keep].abs().max().item()
    assert err <= max(2.0 * yard, 0.02 * want[keep].abs().max().item()), (err, yard)


@pytest.mark.gpu
@pytest.mark.parametrize("name,impl,backend", [("llama", "eager", "flashlight_amd_inductor"), ("gpt2", "eager", "flashlight_amd"),
                                               ("gemma2", "sdpa", "flashlight_amd"), ("gptj", "eager", "flashlight_amd")])
def test_transformers_training_step(name, impl, backend):
    """A language-model loss and its backward through the compiled model: the gradient of every parameter against the
    same model in fp32 on the CPU, with eager bf16 on the GPU as the yardstick."""
    cls, kw, _ = CONFIGS[name]
    if not hasattr(transformers, cls):
        pytest.skip(f"this transformers has no {cls}")
    kw = dict(kw, **({"attn_pdrop": 0.0, "resid_pdrop": 0.0, "embd_pdrop": 0.0} if name in ("gpt2", "gptj") else {}))
    torch.manual_seed(1)
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, 1000, (2, 160), generator=g)
    attend = torch.ones(2, 160, dtype=torch.long)
    attend[1, :30] = 0
    labels = ids.clone()
    labels[attend == 0] = -100
    labels[1, 30] = -100   # predicted from position 29, which attends nothing: arbitrary in any implementation
    model = transformers.AutoModelForCausalLM.from_config(getattr(transformers, cls)(**kw), attn_implementation=impl).train()
    ref = copy.deepcopy(model).float()
    eager = copy.deepcopy(model).to(torch.bfloat16).cuda()
    m = model.to(torch.bfloat16).cuda()
    ref(input_ids=ids, attention_mask=attend, labels=labels).loss.backward()
    eager(input_ids=ids.cuda(), attention_mask=attend.cuda(), labels=labels.cuda()).loss.backward()
    torch._dynamo.reset()
    loss = torch.compile(m, backend=backend, dynamic=False)(input_ids=ids.cuda(), attention_mask=attend.cuda(), labels=labels.cuda()).loss
    loss.backward()
    worst = yard = 0.0
    for (pn, p32), (_, pe), (_, pm) in zip(ref.named_parameters(), eager.named_parameters(), m.named_parameters()):
        if p32.grad is None:
            continue
        assert pm.grad is not None and torch.isfinite(pm.grad).all(), pn
        top = p32.grad.abs().max().item() + 1e-8
        worst = max(worst, (pm.grad.float().cpu() - p32.grad).abs().max().item() / top)
        yard = max(yard, (pe.grad.float().cpu() - p32.grad).abs().max().item() / top)
    assert worst <= max(2.0 * yard, 0.03), (worst, yard)
