"""Transformer blocks around the Fastmax operator: a ViT-style classifier and a decoder-only
language model, enough to run the reference's two training steps (image classification with
4x4 patches + class token, next-token prediction with a causal mask) on this library.

What is mirrored from the reference (``transformer/model.py:252-465``, ``modules.py:6-56``):
three bias-free projections and an output projection per attention layer with the same
parameter names, pre-LayerNorm blocks whose MLP residual adds the block input (``model.py:366``),
learned position embedding with one spare slot for the class token (``model.py:420``), xavier
initialisation of every matrix (``model.py:436-438``), the three classifier heads.

What is done differently: q, k, v stay the transposed views of the projection outputs (the
operator takes batch and head strides and writes its result in the same order, so the head
split and merge cost no copies; the reference makes eight, ``model.py:29-32,46,62,65-67``);
the gradient flows through the q/k normalisation (the reference extension drops it,
``fastmax_cuda_backward.cu`` has no counterpart of ``apply_norm``); the attention arguments
come from the constructor (the reference overrides them with constants at ``model.py:294-305``).
"""
import math

import torch
from torch import nn

from ..attention_mechanisms.score_function import (CENTRE_NONE, FASTMultiHeadAttention_Function, FastmaxDecodeState,
                                                    FastmaxNormalize, FastmaxNormAttention, _fold_possible)


def fastmax_attention(q, k, v, *, mask, normalize, lim, temperature, a0, a1, a2, p):
    """``(b, h, n, d)`` views in, ``(b, h, n, d)`` out, on the HIP kernels."""
    if normalize and _fold_possible(q, k, mask):
        # the normalisation folded into the attention kernels, its gradient included
        return FastmaxNormAttention.apply(q, k, v, bool(mask), float(lim), float(temperature), float(a0), float(a1),
                                          float(a2), int(p))
    if normalize:
        q = FastmaxNormalize.apply(q, CENTRE_NONE, float(lim))
        k = FastmaxNormalize.apply(k, CENTRE_NONE, float(lim))
    return FASTMultiHeadAttention_Function.apply(q, k, v, None, None, bool(mask), 0.0, False, float(temperature),
                                                 float(a0), float(a1), float(a2), float(lim), int(p))


class Attention(nn.Module):
    """Multi-head Fastmax attention (reference ``transformer/model.py:252-338``).
    ``attention_fn`` replaces the kernel call (tests put the CPU oracle there)."""

    def __init__(self, d_model, d_head, h, dropout_rate=0.0, use_masking=False, normalize=True, p=2,
                 temperature=1.0, lim=1.0, coefficients=(1.0, 1.0, 0.5), attention_fn=None):
        super().__init__()
        self.d_head, self.h = d_head, h
        self.use_masking, self.normalize, self.p = use_masking, normalize, p
        self.temperature, self.lim, self.coefficients = temperature, lim, coefficients
        self.attention_fn = attention_fn or fastmax_attention
        self.query_transform = nn.Linear(d_model, h * d_head, bias=False)
        self.key_transform = nn.Linear(d_model, h * d_head, bias=False)
        self.value_transform = nn.Linear(d_model, h * d_head, bias=False)
        self.linear = nn.Linear(h * d_head, d_model)
        self.dropout = nn.Dropout(dropout_rate)

    def forward(self, x, cache=None):
        """``cache``: None, or a dict holding the key and value projections of the tokens seen so far
        (``"k"``, ``"v"``: ``(b, n_past, h*d)``); x then holds only the new tokens, attends to past and
        new keys (causal, queries aligned to the last keys) and the dict is updated in place."""
        b, n, _ = x.shape
        q = self.query_transform(x).view(b, n, self.h, self.d_head).transpose(1, 2)   # (b, h, n, d) views
        kp, vp = self.key_transform(x), self.value_transform(x)
        if cache is not None and self.normalize:
            raise ValueError("cached decoding needs normalize=False: the max-norm scaling looks at every token")
        if cache is not None and cache.get("kind") == "state":
            # O(1) decoding: the layer keeps the moment state instead of the keys and values (needs the causal mask)
            if not self.use_masking:
                raise ValueError("the decoding state is causal attention's; this layer is unmasked")
            if "state" not in cache:
                a0, a1, a2 = self.coefficients
                cache["state"] = FastmaxDecodeState(self.temperature, a0, a1, a2, self.p)
            k = kp.view(b, n, self.h, self.d_head).transpose(1, 2)
            v = vp.view(b, n, self.h, self.d_head).transpose(1, 2)
            st = cache["state"]
            o = st.step(q, k, v) if (n == 1 and st.tokens) else st.prompt(q, k, v)
            cache["n"] = st.tokens
            o = o.transpose(1, 2).reshape(b, n, self.h * self.d_head)
            return self.dropout(self.linear(o))
        if cache is not None:
            cache["n"] = cache.get("n", 0) + n
            if "k" in cache:
                kp, vp = torch.cat((cache["k"], kp), dim=1), torch.cat((cache["v"], vp), dim=1)
            cache["k"], cache["v"] = kp, vp
        nk = kp.shape[1]
        k = kp.view(b, nk, self.h, self.d_head).transpose(1, 2)
        v = vp.view(b, nk, self.h, self.d_head).transpose(1, 2)
        a0, a1, a2 = self.coefficients
        o = self.attention_fn(q, k, v, mask=self.use_masking, normalize=self.normalize, lim=self.lim,
                              temperature=self.temperature, a0=a0, a1=a1, a2=a2, p=self.p)
        o = o.transpose(1, 2).reshape(b, n, self.h * self.d_head)                     # a view when o is (b, n, h, d) in memory
        return self.dropout(self.linear(o))


class TransformerBlock(nn.Module):
    """Attention + MLP, pre-LayerNorm (reference ``transformer/model.py:340-370``)."""

    def __init__(self, num_heads, d_model, d_mlp, dropout_rate=0.0, **attention_args):
        super().__init__()
        self.layer_norm1 = nn.LayerNorm(d_model)
        self.attention_subblock = Attention(d_model, d_model // num_heads, num_heads, dropout_rate, **attention_args)
        self.layer_norm2 = nn.LayerNorm(d_model)
        self.mlp_subblock = nn.Sequential(nn.Linear(d_model, d_mlp), nn.GELU(), nn.Linear(d_mlp, d_model),
                                          nn.Dropout(dropout_rate))

    def forward(self, x, cache=None):
        a = self.attention_subblock(self.layer_norm1(x), cache) + x
        # the reference adds the block input, not the attention output, to the MLP branch (model.py:366)
        return self.mlp_subblock(self.layer_norm2(a)) + x


class ConvEmbedding(nn.Module):
    """Non-overlapping patches through one convolution (reference ``modules.py:45-56``)."""

    def __init__(self, channels, patch_shape, d_model):
        super().__init__()
        self.conv = nn.Conv2d(channels, d_model, kernel_size=patch_shape, stride=patch_shape)

    def forward(self, images):
        return self.conv(images).flatten(2).transpose(1, 2)          # (b, n, d_model)


class _Head(nn.Module):
    """LayerNorm + Linear on every token, the first token, or the token average
    (reference ``modules.py:6-43``)."""

    def __init__(self, d_model, n_out, kind):
        super().__init__()
        self.kind = kind
        self.layer_norm = nn.LayerNorm(d_model)
        self.linear = nn.Linear(d_model, n_out)

    def forward(self, x):
        x = self.layer_norm(x)
        if self.kind == "cls_token":
            x = x[:, 0, :]
        elif self.kind == "avg_pool":
            x = x.mean(dim=1)
        return self.linear(x)


class Transformer(nn.Module):
    """Reference ``transformer/model.py:373-465`` with ``embedding`` in {"discrete_set", "patch_conv"}
    and ``classifier`` in {"per_token", "avg_pool", "cls_token"}.  ``forward`` returns the logits."""

    def __init__(self, out_dim, max_tokens, d_model=512, d_mlp=2048, heads_per_block=8, num_blocks=6, dropout_rate=0.0,
                 use_masking=False, embedding="discrete_set", classifier="per_token", vocab_size=None, patch_shape=None,
                 patch_channels=None, normalize=True, p=2, temperature=1.0, lim=1.0, attention_fn=None):
        super().__init__()
        if embedding == "discrete_set":
            self.token_embedding = nn.Embedding(vocab_size, d_model)
        elif embedding == "patch_conv":
            self.token_embedding = ConvEmbedding(patch_channels, patch_shape, d_model)
        else:
            raise ValueError(f"Unknown embedding type: {embedding}")
        self.pos_embedding = nn.Embedding(max_tokens + 1, d_model)
        self.blocks = nn.ModuleList(
            TransformerBlock(heads_per_block, d_model, d_mlp, dropout_rate, use_masking=use_masking, normalize=normalize,
                             p=p, temperature=temperature, lim=lim, attention_fn=attention_fn)
            for _ in range(num_blocks))
        if classifier not in ("per_token", "avg_pool", "cls_token"):
            raise ValueError(f"Unknown classifier type: {classifier}")
        if classifier == "cls_token":
            self.class_token = nn.Parameter(torch.randn(d_model))
        self.classifier = _Head(d_model, out_dim, classifier)
        for prm in self.parameters():
            if prm.dim() > 1:
                nn.init.xavier_uniform_(prm)

    def forward(self, tokens, caches=None):
        """``caches``: None, or one dict per block (see ``Attention.forward``); ``tokens`` then holds
        only the tokens that follow the cached ones."""
        x = self.token_embedding(tokens)
        if self.classifier.kind == "cls_token":
            x = torch.cat((self.class_token.expand(x.shape[0], 1, -1), x), dim=1)
        past = caches[0].get("n", 0) if caches else 0
        x = x + self.pos_embedding(torch.arange(past, past + x.shape[1], device=x.device))
        for i, block in enumerate(self.blocks):
            x = block(x, caches[i] if caches is not None else None)
        return self.classifier(x)

    @torch.no_grad()
    def generate(self, tokens, max_new_tokens, sample=False, use_cache=True):
        """Next-token generation (reference ``transformer/eval.py:8-32``): ``tokens`` ``(b, n)`` grows
        by ``max_new_tokens``.  The reference runs the whole context through the model for every
        new token.  With ``use_cache="state"`` every layer keeps the O(1) moment state of its keys and values
        (``FastmaxDecodeState``) and a step costs the same whatever the context length; with
        ``use_cache=True`` the key and value projections of every block are kept and a
        step runs the new token only; its attention is one causal call with one query and all the
        keys so far.  That is exact for ``normalize=False`` models (the max-norm scaling of the
        others depends on every token, so they take the reference's route).  Contexts longer than
        the position table are not handled (the reference crops to the last ``max_tokens``)."""
        cached = bool(use_cache) and not any(b.attention_subblock.normalize for b in self.blocks)
        # use_cache = "state": every layer keeps its O(1) moment state (the prompt goes through ordinary causal
        # attention once and is absorbed); True: keys and values are kept and re-read every step
        kind = "state" if use_cache == "state" else "kv"
        caches = [dict(kind=kind) for _ in self.blocks] if cached else None
        logits = self(tokens, caches)[:, -1, :]
        for _ in range(max_new_tokens):
            nxt = torch.multinomial(torch.softmax(logits, -1), 1) if sample else logits.argmax(-1, keepdim=True)
            tokens = torch.cat((tokens, nxt), dim=1)
            logits = (self(nxt, caches) if cached else self(tokens))[:, -1, :]
        return tokens


def vit_for_c4(**overrides):
    """The image-classification configuration of the reference's lightning script at MNIST scale:
    28x28 one-channel images, 4x4 patches (49 tokens + class token), d_model 128, 4 layers,
    4 heads of 32, 10 classes."""
    cfg = dict(out_dim=10, max_tokens=49, d_model=128, d_mlp=512, heads_per_block=4, num_blocks=4, use_masking=False,
               embedding="patch_conv", classifier="cls_token", patch_shape=(4, 4), patch_channels=1, normalize=True, p=2)
    cfg.update(overrides)
    return Transformer(**cfg)


def gpt_for_c5(**overrides):
    """Decoder-only language model: 6 layers, d_model 512, 8 heads of 64, context 1024, GPT-2
    vocabulary size."""
    cfg = dict(out_dim=50257, max_tokens=1024, d_model=512, d_mlp=2048, heads_per_block=8, num_blocks=6,
               use_masking=True, embedding="discrete_set", classifier="per_token", vocab_size=50257, normalize=True, p=2)
    cfg.update(overrides)
    return Transformer(**cfg)
