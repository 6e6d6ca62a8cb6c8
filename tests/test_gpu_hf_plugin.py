"""The attention plug-in driven the way the reference drives it: HF attention modules whose
config names the HIP implementation look it up in HF's global attention registry
(models/attention.py:107-108, models/eagle3/core.py:49-60, models/dflash/model_definitions.py:134-152)
and pass the mask object through untouched.  Output and gradients against the same HF module on
its eager path under the oracle's dense mask."""

import pytest
import torch

from oracle import masks as OM

pytestmark = pytest.mark.gpu


def _rel(got, want):
    return (got.float() - want.float()).abs().max().item() / (want.float().abs().max().item() + 1e-12)


@pytest.mark.parametrize("hq,hkv,d,window", [(4, 2, 64, None), (8, 1, 128, 24)])
def test_hf_llama_attention_dispatches_to_ttt_hip(hq, hkv, d, window):
    from transformers import DynamicCache, LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaAttention, LlamaRotaryEmbedding

    from speculators_amd import attention as A

    A.register_with_transformers()
    h, t, steps = 256, 200, 3
    cfg = LlamaConfig(hidden_size=h, num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d,
                      intermediate_size=512, vocab_size=128, num_hidden_layers=1, attention_bias=False,
                      rope_parameters={"rope_type": "default", "rope_theta": 10000.0})
    torch.manual_seed(0)
    cfg._attn_implementation = "eager"
    ref_attn = LlamaAttention(cfg, 0).to(torch.bfloat16).cuda()
    hip_cfg = LlamaConfig(**cfg.to_dict())
    hip_cfg._attn_implementation = A.ATTN_IMPL_TTT
    hip_attn = LlamaAttention(hip_cfg, 0).to(torch.bfloat16).cuda()
    hip_attn.load_state_dict(ref_attn.state_dict())
    rot = LlamaRotaryEmbedding(cfg).cuda()

    doc = torch.tensor([0] * 90 + [1] * 100 + [-1] * 10)
    pos = torch.cat([1 + torch.arange(90), 1 + torch.arange(100), torch.zeros(10, dtype=torch.long)])[None].cuda()
    mask = A.create_ttt_mask(doc.cuda(), t, window)
    g = torch.Generator().manual_seed(1)
    cache_ref, cache_hip = DynamicCache(), DynamicCache()
    outs_ref, outs_hip, xs_ref, xs_hip = [], [], [], []
    for step in range(steps):
        x = torch.randn(1, t, h, generator=g).bfloat16().cuda()
        xr, xh = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
        cos, sin = rot(x, pos + step)
        dense = OM.ttt_mask_dense(doc, t, step, window).cuda()
        fmask = torch.zeros(1, 1, t, (step + 1) * t, device="cuda", dtype=torch.bfloat16).masked_fill(
            ~dense[None, None], float("-inf"))
        o_ref, _ = ref_attn(hidden_states=xr, position_embeddings=(cos, sin), attention_mask=fmask,
                            past_key_values=cache_ref)
        o_hip, w_hip = hip_attn(hidden_states=xh, position_embeddings=(cos, sin), attention_mask=mask,
                                past_key_values=cache_hip)
        assert w_hip is None and o_hip.shape == o_ref.shape
        assert _rel(o_hip, o_ref) <= 2e-2, step
        outs_ref.append(o_ref), outs_hip.append(o_hip), xs_ref.append(xr), xs_hip.append(xh)
        mask = mask.extended()
    go = [torch.randn(1, t, h, generator=g).bfloat16().cuda() for _ in range(steps)]
    torch.autograd.backward(outs_ref, go)
    torch.autograd.backward(outs_hip, go)
    for step in range(steps):  # the keys of step j also receive gradient from the later steps' queries
        assert _rel(xs_hip[step].grad, xs_ref[step].grad) <= 3e-2, step
    for (n, p_ref), (_, p_hip) in zip(ref_attn.named_parameters(), hip_attn.named_parameters(), strict=True):
        assert _rel(p_hip.grad, p_ref.grad) <= 3e-2, n


def test_wrong_mask_object_is_refused():
    from speculators_amd import attention as A

    q = torch.zeros(1, 2, 8, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(TypeError, match="TTTMask"):
        A.ttt_hip_attention_forward(None, q, q, q, torch.zeros(8, 8, device="cuda"))
    with pytest.raises(TypeError, match="DFlashMask"):
        A.dflash_hip_attention_forward(None, q, q, q, None)


@pytest.mark.parametrize("window,non_causal", [(None, False), (6, False), (6, True)])
def test_hf_blocks_wired_like_qwen3_dflash_attention_dispatch_to_dflash_hip(window, non_causal):
    from hf_blocks import HFDFlashLayer, qwen3_cfg
    from transformers.models.qwen3.modeling_qwen3 import Qwen3RotaryEmbedding

    from oracle import dflash as OD
    from oracle.eagle3 import DraftShape
    from speculators_amd import attention as A

    A.register_with_transformers()
    shape = DraftShape(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
                       intermediate_size=512, vocab_size=50, draft_vocab_size=20, num_aux=2,
                       num_hidden_layers=1, qk_norm=True, rms_norm_eps=1e-6, rope_theta=10000.0)
    w = OD.random_weights(shape, 0, std=0.05)
    g = torch.Generator().manual_seed(3)
    for name in list(w):
        if name.endswith("norm.weight") or "layernorm" in name:
            w[name] = 1 + 0.2 * torch.randn(w[name].shape, generator=g)
    cfg = qwen3_cfg(shape)
    t, bs = 40, 4
    doc = torch.tensor([0] * 22 + [1] * 14 + [-1] * 4)
    pos = torch.cat([torch.arange(22), torch.arange(14), torch.zeros(4, dtype=torch.long)])[None]
    anchors = torch.tensor([3, 9, 17, 25, 30, 0])
    noise = torch.randn(1, anchors.numel() * bs, shape.hidden_size, generator=g).bfloat16().cuda()
    ctx = torch.randn(1, t, shape.hidden_size, generator=g).bfloat16().cuda()
    bpos = (pos[0, anchors][:, None] + torch.arange(bs)[None]).reshape(1, -1)
    cos, sin = Qwen3RotaryEmbedding(cfg).cuda()(ctx, torch.cat([pos, bpos], 1).cuda())
    dense = OM.dflash_mask_dense(doc, t, anchors, bs, window, non_causal).cuda()
    desc = A.create_dflash_mask(doc.cuda(), t, anchors.cuda(), bs, window, non_causal)
    ref_layer = HFDFlashLayer(cfg, w, 0, "eager").to(torch.bfloat16).cuda()
    hip_layer = HFDFlashLayer(cfg, w, 0, A.ATTN_IMPL_DFLASH).to(torch.bfloat16).cuda()
    go = torch.randn(noise.shape, generator=g).bfloat16().cuda()
    res = []
    for layer, m in ((ref_layer, dense), (hip_layer, desc)):
        x, c = noise.clone().requires_grad_(True), ctx.clone().requires_grad_(True)
        out = layer(x, c, cos, sin, m)
        out.backward(go)
        res.append((out.detach(), x.grad, c.grad, {n: p.grad for n, p in layer.named_parameters()}))
    assert _rel(res[1][0], res[0][0]) <= 2e-2
    assert _rel(res[1][1], res[0][1]) <= 3e-2 and _rel(res[1][2], res[0][2]) <= 3e-2
    for n, gr in res[0][3].items():
        assert _rel(res[1][3][n], gr) <= 3e-2, n
