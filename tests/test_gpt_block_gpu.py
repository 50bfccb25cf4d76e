"""The attention operator inside its caller: a small GPT (RoPE on q/k, Fastmax causal attention
in every layer, as reference model.py:464-603 wires it) must train the same way on the HIP
kernels as on the pure-PyTorch path."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
KERNEL_PATH = "auto"   # (conftest) the library's own choice of kernels; the config-5 tests also pin each family


def _hip_attention(layout):
    import bench_gpt
    from fastmax_amd import FASTMultiHeadAttention

    return bench_gpt.PackedAttention() if layout == "packed" else FASTMultiHeadAttention(use_custom_gradient=True)


@pytest.mark.parametrize("p,layout", [(1, "split"), (2, "split"), (1, "packed"), (2, "packed")])
def test_small_gpt_gradients_match_pytorch_path(built, p, layout):
    """layout "split": contiguous q, k, v from the fused split + RoPE kernel; "packed": RoPE in place and
    the attention on strided views of the packed projection, token-major output, gradients written
    straight into the projection's gradient."""
    import bench_gpt
    from fastmax_amd import FASTMultiHeadAttention

    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    ref_model = bench_gpt.MiniGPT(512, 128, 2, 2, 256, 300, FASTMultiHeadAttention(use_custom_gradient=False), p, "pytorch").to(dev)
    hip_model = bench_gpt.MiniGPT(512, 128, 2, 2, 256, 300, _hip_attention(layout), p, layout).to(dev)
    hip_model.load_state_dict(ref_model.state_dict())
    idx = torch.randint(0, 512, (2, 301), device=dev, generator=torch.Generator(device=dev).manual_seed(1))
    x, y = idx[:, :-1].contiguous(), idx[:, 1:].contiguous()
    losses = []
    for m in (ref_model, hip_model):
        logits = m(x)
        loss = F.cross_entropy(logits.view(-1, 512), y.view(-1))
        loss.backward()
        losses.append(float(loss.detach()))
    assert abs(losses[0] - losses[1]) <= 1e-5 * abs(losses[0])
    for (name, a), (_, b) in zip(ref_model.named_parameters(), hip_model.named_parameters()):
        err = float((a.grad - b.grad).norm() / a.grad.norm().clamp_min(1e-30))
        assert err <= 1e-3, (name, err)


class _Fp32PyTorchAttention(torch.nn.Module):
    """The pure-PyTorch function on the same bf16-rounded q, k, v, evaluated in fp32 outside
    autocast: what the kernels (bf16 in, fp32 accumulation, bf16 out) are specified against."""

    def forward(self, q, k, v, drop_noise, mask, dropout, normalize, temperature, a0, a1, a2, lim, p):
        from fastmax_amd import fastmax_function

        with torch.autocast("cuda", enabled=False):
            o = fastmax_function(q.float(), k.float(), v.float(), mask, dropout, normalize, temperature,
                                 a0, a1, a2, lim, p)
        return o.to(q.dtype)


@pytest.mark.parametrize("path", ["auto", "moments"])
@pytest.mark.parametrize("p,layout", [(2, "split"), (1, "split"), (2, "packed"), (1, "packed")])
def test_gpt_at_config5_widths_bf16_gradients(built, monkeypatch, p, layout, path):
    """d_model 768, 12 heads x 64, MLP 3072, T = 2048, bf16 autocast, fused projection split + RoPE
    (two layers, batch 2, a small vocabulary): loss and every parameter gradient of the model on the
    HIP kernels against the same model with the PyTorch attention function, at the bf16 tolerance."""
    import bench_gpt
    from fastmax_amd import FASTMultiHeadAttention

    if path == "moments":   # (auto takes the dense kernels at this length: score tiles for p = 2, their linear mode for p = 1)
        monkeypatch.setenv("FASTMAX_PATH", "moments")
    dev = torch.device("cuda:0")
    vocab, T = 1024, 2048
    torch.manual_seed(0)
    ref_model = bench_gpt.MiniGPT(vocab, 768, 2, 12, 3072, T, _Fp32PyTorchAttention(), p, "pytorch").to(dev)
    hip_model = bench_gpt.MiniGPT(vocab, 768, 2, 12, 3072, T, _hip_attention(layout), p, layout).to(dev)
    hip_model.load_state_dict(ref_model.state_dict())
    idx = torch.randint(0, vocab, (2, T + 1), device=dev, generator=torch.Generator(device=dev).manual_seed(3))
    x, y = idx[:, :-1].contiguous(), idx[:, 1:].contiguous()
    losses = []
    for m in (ref_model, hip_model):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits = m(x)
        loss = F.cross_entropy(logits.float().view(-1, vocab), y.view(-1))
        loss.backward()
        losses.append(float(loss.detach()))
    print("losses", losses, flush=True)
    assert abs(losses[0] - losses[1]) <= 2e-3 * abs(losses[0])
    worst = ("", 0.0)
    for (name, a), (_, b) in zip(ref_model.named_parameters(), hip_model.named_parameters()):
        err = float((a.grad.double() - b.grad.double()).norm() / a.grad.double().norm().clamp_min(1e-30))
        print(name, f"{err:.3e}", flush=True)
        if err > worst[1]:
            worst = (name, err)
    assert worst[1] <= 2e-2, worst


def test_bf16_autocast_step_runs_and_learns(built):
    import bench_gpt
    from fastmax_amd import FASTMultiHeadAttention

    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    model = bench_gpt.MiniGPT(512, 128, 2, 2, 256, 256, bench_gpt.PackedAttention(), 2, "packed").to(dev)
    opt = torch.optim.AdamW(model.parameters(), lr=1e-3)
    idx = torch.randint(0, 512, (4, 257), device=dev, generator=torch.Generator(device=dev).manual_seed(2))
    x, y = idx[:, :-1].contiguous(), idx[:, 1:].contiguous()
    losses = []
    for _ in range(8):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits = model(x)
        loss = F.cross_entropy(logits.float().view(-1, 512), y.view(-1))
        opt.zero_grad(set_to_none=True)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert all(v == v for v in losses) and losses[-1] < losses[0]


@pytest.mark.parametrize("path,p", [("auto", 2), ("moments", 2), ("auto", 1)])
def test_config5_full_depth_step(built, monkeypatch, path, p):
    """One forward + backward of the whole configuration-5 model -- 12 layers, d_model 768, 12 heads x 64,
    MLP 3072, RoPE, vocabulary 50304, batch 8, T = 2048, bf16 autocast -- on the HIP kernels (the library's
    own choice, which is the dense score tiles at this length -- at p = 1, the order the reference model sets
    (model.py:212), their linear mode -- and the moment kernels): finite loss near ln(vocabulary) for random
    weights, finite gradients in every parameter, none of them all zero."""
    import math

    import bench_gpt

    if path == "moments":
        monkeypatch.setenv("FASTMAX_PATH", "moments")
    dev = torch.device("cuda:0")
    vocab, T, B = 50304, 2048, 8
    torch.manual_seed(0)
    model = bench_gpt.MiniGPT(vocab, 768, 12, 12, 3072, T, bench_gpt.PackedAttention(), p, "packed").to(dev)
    idx = torch.randint(0, vocab, (B, T + 1), device=dev, generator=torch.Generator(device=dev).manual_seed(4))
    x, y = idx[:, :-1].contiguous(), idx[:, 1:].contiguous()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        logits = model(x)
    loss = F.cross_entropy(logits.float().view(-1, vocab), y.view(-1))
    loss.backward()
    lv = float(loss.detach())
    print("loss", lv, flush=True)
    assert math.isfinite(lv) and abs(lv - math.log(vocab)) < 0.5
    for name, prm in model.named_parameters():
        assert prm.grad is not None and bool(torch.isfinite(prm.grad).all()), name
        assert float(prm.grad.abs().max()) > 0.0, name
    del model, logits, loss
    torch.cuda.empty_cache()
