"""The synthetic decoder driver on a tiny configuration: the captured decode step equals the
eager one, and a decode step continues a prefill the way a longer prefill would."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _tiny(sba):
    from importlib import import_module
    dec = import_module(sba.__name__ + ".decoder")
    cfg = dec.DecoderConfig(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=64, experts=8, topk=2,
                            inter=128, vocab=1000, group=128)
    return dec, cfg


def test_graph_decode_equals_eager(sba, gpu):
    dec, cfg = _tiny(sba)
    gen = torch.Generator(device=gpu).manual_seed(5)
    ids = torch.randint(0, cfg.vocab, (8, 24), device=gpu, generator=gen)
    outs = []
    for use_graph in (False, True):
        m = dec.SyntheticMoEDecoder(cfg, 8, 40, gpu, seed=11)
        m.prefill(ids, chunk_seqs=3)
        if use_graph:
            pos, tok = m.pos.clone(), m.tok.clone()
            m.capture()
            m.pos.copy_(pos); m.tok.copy_(tok)
        outs.append(m.decode(12, use_graph).cpu())
    assert torch.equal(outs[0], outs[1])


def test_decode_step_continues_prefill(sba, gpu):
    dec, cfg = _tiny(sba)
    gen = torch.Generator(device=gpu).manual_seed(6)
    ids = torch.randint(0, cfg.vocab, (8, 33), device=gpu, generator=gen)
    a = dec.SyntheticMoEDecoder(cfg, 8, 40, gpu, seed=12)
    a.prefill(ids[:, :32])
    a.tok.copy_(ids[:, 32])            # force the known 33rd token
    a.decode(1, use_graph=False)
    b = dec.SyntheticMoEDecoder(cfg, 8, 40, gpu, seed=12)
    b.prefill(ids)
    la, lb = a.last_logits.float(), b.last_logits.float()
    err = float((la - lb).norm() / lb.norm())
    print(f"[decoder] decode-vs-prefill logits rel_fro={err:.2e}", flush=True)
    assert err <= 2e-2
    assert (a.next_tok == b.tok).float().mean().item() >= 0.75


def test_full_width_layer_awq_ops_against_dequant_matmul(sba, gpu):
    """One Qwen3-30B-A3B-width layer (hidden 2048, 32 / 4 heads of 128, 128 experts, top-8,
    intermediate 768): an 8192-token prefill pass (64 prompts of 128 tokens in one chunk) and a
    decode step at batch 64, with the output of every AWQ call (qkv, o, MoE block) compared with
    the dequantize kernel + library matmul / dense expert evaluation on the same input."""
    from importlib import import_module
    dec = import_module(sba.__name__ + ".decoder")
    cfg = dec.DecoderConfig(layers=1, vocab=4096)
    m = dec.SyntheticMoEDecoder(cfg, 64, 130, gpu, seed=21)
    ids = torch.randint(0, cfg.vocab, (64, 128), device=gpu, generator=torch.Generator(device=gpu).manual_seed(22))
    chk = dec.AwqOpChecker(cfg.topk)
    m.checker = chk
    m.prefill(ids, chunk_seqs=64)
    prefill_worst = dict(chk.worst)
    assert chk.calls == 3
    m.decode(1, use_graph=False)
    assert chk.calls == 6
    print(f"[decoder full width] prefill {prefill_worst} decode-or-prefill max {chk.worst}", flush=True)
    assert set(chk.worst) == {"qkv", "o", "moe"}
    assert max(chk.worst.values()) <= 2e-3
