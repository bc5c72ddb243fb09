"""Model counterparts: the HIP operator against the CPU oracle inside the same model with the same
weights - loss and every parameter gradient must agree (the reference's own model files cannot run
here: they import kornia, lightning and the CUDA extension)."""
import copy

import pytest
import torch

from oracle import fastmax_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def oracle_attention(q, k, v, *, mask, normalize, lim, temperature, a0, a1, a2, p):
    """Closed form in float64 with torch autograd through the normalisation as well."""
    dt = q.dtype
    q, k, v = q.double(), k.double(), v.double()
    if normalize:
        q, k = O.normalize_lim(q, lim), O.normalize_lim(k, lim)
    o, _ = O.closed_form_forward(q, k, v, mask=mask, tau=float(temperature), p=p, a0=a0, a1=a1, a2=a2)
    return o.to(dt)


def grads_of(model, loss):
    model.zero_grad(set_to_none=True)
    loss.backward()
    return {n: p.grad.detach().double().cpu() for n, p in model.named_parameters()}


def compare(model_hip, model_ref, inputs, target, loss_fn, tol_loss, tol_grad):
    out_h = model_hip(inputs)
    out_r = model_ref(inputs)
    lh, lr = loss_fn(out_h, target), loss_fn(out_r, target)
    assert abs(lh.item() - lr.item()) <= tol_loss * max(1.0, abs(lr.item())), (lh.item(), lr.item())
    gh, gr = grads_of(model_hip, lh), grads_of(model_ref, lr)
    assert gh.keys() == gr.keys()
    worst = 0.0
    for name in gr:
        err = float((gh[name] - gr[name]).norm() / max(float(gr[name].norm()), 1e-6))
        worst = max(worst, err)
        assert err < tol_grad, f"{name}: {err:.3e}"
    return lh.item(), worst


def test_vit_step_matches_oracle_fp32():
    from reproducing_fastmax_results_amd.transformer.model import vit_for_c4
    torch.manual_seed(3)
    hip = vit_for_c4(num_blocks=2).to(DEV)
    ref = copy.deepcopy(hip)
    for blk in ref.blocks:
        blk.attention_subblock.attention_fn = oracle_attention
    images = torch.rand(8, 1, 28, 28, generator=torch.Generator().manual_seed(3)).to(DEV)
    labels = torch.randint(0, 10, (8,), generator=torch.Generator().manual_seed(4)).to(DEV)
    loss, worst = compare(hip, ref, images, labels, torch.nn.functional.cross_entropy, 1e-5, 2e-4)
    print(f"vit fp32: loss {loss:.5f}, worst parameter-gradient rel-L2 {worst:.2e}", flush=True)


def test_gpt_step_matches_oracle_bf16():
    from reproducing_fastmax_results_amd.transformer.model import gpt_for_c5
    torch.manual_seed(4)
    hip = gpt_for_c5(num_blocks=2, vocab_size=512, out_dim=512, max_tokens=300).to(DEV).to(torch.bfloat16)
    ref = copy.deepcopy(hip)
    for blk in ref.blocks:
        blk.attention_subblock.attention_fn = oracle_attention
    tokens = torch.randint(0, 512, (2, 300), generator=torch.Generator().manual_seed(5)).to(DEV)
    target = torch.randint(0, 512, (2, 300), generator=torch.Generator().manual_seed(6)).to(DEV)

    def lm_loss(logits, tgt):
        return torch.nn.functional.cross_entropy(logits.float().view(-1, logits.shape[-1]), tgt.view(-1))

    loss, worst = compare(hip, ref, tokens, target, lm_loss, 2e-2, 6e-2)
    print(f"gpt bf16: loss {loss:.4f}, worst parameter-gradient rel-L2 {worst:.2e}", flush=True)


def test_attention_layout_needs_no_copies():
    """The head split and merge around the operator are views (batch and head strides)."""
    from reproducing_fastmax_results_amd.transformer.model import Attention
    att = Attention(128, 32, 4, use_masking=True).to(DEV)
    seen = {}

    def spy(q, k, v, **kw):
        from reproducing_fastmax_results_amd.transformer.model import fastmax_attention
        o = fastmax_attention(q, k, v, **kw)
        seen["q_view"] = q._base is not None and not q.is_contiguous()
        seen["o_merge_is_view"] = o.transpose(1, 2).is_contiguous()
        return o

    att.attention_fn = spy
    y = att(torch.randn(2, 70, 128, device=DEV))
    assert y.shape == (2, 70, 128) and seen["q_view"] and seen["o_merge_is_view"]


def test_cached_generation_matches_full_recompute():
    """Greedy next-token generation with cached keys and values (one causal call with one query and
    all keys so far per block and step) against the reference's loop that runs the whole context for
    every token (transformer/eval.py:8-32), and the step logits against the oracle inside the model."""
    from reproducing_fastmax_results_amd.transformer.model import gpt_for_c5
    torch.manual_seed(5)
    cfg = dict(out_dim=97, vocab_size=97, max_tokens=96, d_model=128, d_mlp=256, heads_per_block=4, num_blocks=2,
               normalize=False, temperature=8.0 * 32 ** 0.5)
    hip = gpt_for_c5(**cfg).to(DEV).eval()
    prompt = torch.randint(0, 97, (3, 40), generator=torch.Generator().manual_seed(6)).to(DEV)
    fast = hip.generate(prompt, 24, use_cache=True)
    slow = hip.generate(prompt, 24, use_cache=False)
    assert fast.shape == (3, 64) and torch.equal(fast[:, :40], prompt)
    assert torch.equal(fast, slow)
    # logits of one cached step against the oracle's full forward over the same tokens
    ref = copy.deepcopy(hip)
    for blk in ref.blocks:
        blk.attention_subblock.attention_fn = oracle_attention
    with torch.no_grad():
        caches = [dict() for _ in hip.blocks]
        hip(fast[:, :50], caches)
        step = hip(fast[:, 50:51], caches)[:, -1, :]
        want = ref(fast[:, :51])[:, -1, :]
    assert float((step - want).norm() / want.norm()) < 1e-4
    # models that normalise q and k cannot cache (the scaling sees every token): same route as the reference
    norm_model = gpt_for_c5(**dict(cfg, normalize=True, temperature=1.0)).to(DEV).eval()
    assert norm_model.generate(prompt, 3).shape == (3, 43)

