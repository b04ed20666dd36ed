"""ToyNSALlama on the GPU: cached inference (prefill + greedy decode steps) reproduces the logits of the training
forward on the extended sequences, and a training step produces finite gradients everywhere."""
import pytest
import torch

from native_sparse_attention.model import InferenceConfig, ToyNSALlama, ToyNSALlamaConfig
from native_sparse_attention.testing import cu_from_lens

pytestmark = pytest.mark.gpu


def _model(device):
    torch.manual_seed(0)
    cfg = ToyNSALlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=8,
                            num_key_value_heads=2, head_dim=64, topk=4, window_size=512)
    return ToyNSALlama(cfg, InferenceConfig(max_batch_size=3, max_length=512, max_new_tokens=4), device=device).to(device).bfloat16()


def test_generate_matches_training_forward(device):
    model = _model(device).eval()
    lens = [150, 60, 333]
    cu = cu_from_lens(lens, device)
    g = torch.Generator(device=device).manual_seed(1)
    prompt = torch.randint(0, 512, (int(cu[-1]),), generator=g, device=device)
    new = model.generate(prompt, cu, 4)
    assert new.shape == (3, 4)
    # teacher forcing: the full forward over prompt + generated tokens must give the same next-token logits
    seqs, s0 = [], 0
    for b, L in enumerate(lens):
        seqs.append(torch.cat([prompt[s0:s0 + L], new[b, :3]]))
        s0 += L
    full_cu = cu_from_lens([L + 3 for L in lens], device)
    with torch.no_grad():
        logits = model(torch.cat(seqs), full_cu)
    model.kv_cache = None
    step_logits = [model.inference(prompt, cu, 0)]
    for step in range(1, 4):
        step_logits.append(model.inference(new[:, step - 1], cu, step))
    for b, L in enumerate(lens):
        for step in range(4):
            want = logits[int(full_cu[b]) + L - 1 + step]
            got = step_logits[step][b]
            assert (got - want).abs().max() < 0.05 * max(1.0, want.abs().max().item()), (b, step)


def test_training_step(device):
    model = _model(device)
    cu = cu_from_lens([200, 100], device)
    ids = torch.randint(0, 512, (300,), device=device)
    logits = model(ids, cu)
    assert logits.shape == (300, 512) and logits.dtype == torch.float32
    loss = torch.nn.functional.cross_entropy(logits[:-1], ids[1:])
    loss.backward()
    for name, p in model.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all(), name


def test_dense_toy_llama_generate_matches_training_forward(device):
    """The dense twin (SelfAttention + KVCache): cached prefill and decode steps against the training forward."""
    from native_sparse_attention.model import ToyLlama, ToyLlamaConfig
    torch.manual_seed(0)
    cfg = ToyLlamaConfig(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=8,
                         num_key_value_heads=2, head_dim=64)
    model = ToyLlama(cfg, InferenceConfig(max_batch_size=3, max_length=512, max_new_tokens=4), device=device).to(device).bfloat16().eval()
    lens = [150, 60, 333]
    cu = cu_from_lens(lens, device)
    g = torch.Generator(device=device).manual_seed(1)
    prompt = torch.randint(0, 512, (int(cu[-1]),), generator=g, device=device)
    new = model.generate(prompt, cu, 4)
    seqs, s0 = [], 0
    for b, L in enumerate(lens):
        seqs.append(torch.cat([prompt[s0:s0 + L], new[b, :3]]))
        s0 += L
    full_cu = cu_from_lens([L + 3 for L in lens], device)
    with torch.no_grad():
        logits = model(torch.cat(seqs), full_cu)
    model.kv_cache = None
    step_logits = [model.inference(prompt, cu, 0)]
    for step in range(1, 4):
        step_logits.append(model.inference(new[:, step - 1], cu, step))
    for b, L in enumerate(lens):
        for step in range(4):
            want = logits[int(full_cu[b]) + L - 1 + step]
            assert (step_logits[step][b] - want).abs().max() < 0.05 * max(1.0, want.abs().max().item()), (b, step)
    loss = torch.nn.functional.cross_entropy(model(prompt, cu)[:-1], prompt[1:])
    loss.backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())
