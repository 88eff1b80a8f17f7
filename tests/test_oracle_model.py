"""Pins oracle/t5_model.py (restates reference modeling.py / attentions.py 'basic') against the
installed HuggingFace T5 implementation (third-party library) on a tiny random model."""
import pytest
import torch

from oracle import t5_model as OM
from turbot5_amd.config import T5Config


@pytest.fixture(scope="module")
def tiny():
    from transformers import T5Config as HFConfig, T5ForConditionalGeneration
    torch.manual_seed(0)
    hf_cfg = HFConfig(vocab_size=100, d_model=32, d_kv=8, d_ff=64, num_layers=2, num_decoder_layers=2, num_heads=4,
                      relative_attention_num_buckets=32, relative_attention_max_distance=128, dropout_rate=0.0,
                      feed_forward_proj="relu", tie_word_embeddings=True, decoder_start_token_id=0)
    hf = T5ForConditionalGeneration(hf_cfg).eval()
    with torch.no_grad():
        for p in hf.parameters():          # HF's default init is tiny for some tensors: make every path matter
            p.copy_(torch.randn_like(p) * 0.3)
    cfg = T5Config(vocab_size=100, d_model=32, d_kv=8, d_ff=64, num_layers=2, num_heads=4, dropout_rate=0.0)
    sd = {k: v.detach().clone() for k, v in hf.state_dict().items()}
    sd["lm_head.weight"] = sd["shared.weight"]
    return hf, cfg, sd


def test_encoder_matches_huggingface(tiny):
    hf, cfg, sd = tiny
    ids = torch.randint(0, 100, (3, 150), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        want = hf.encoder(input_ids=ids).last_hidden_state
    got = OM.encoder_forward(sd, cfg, ids)
    assert torch.allclose(got, want, atol=2e-4, rtol=1e-4)


def test_encoder_with_padding_matches_huggingface(tiny):
    hf, cfg, sd = tiny
    ids = torch.randint(0, 100, (2, 40), generator=torch.Generator().manual_seed(2))
    mask = torch.ones(2, 40)
    mask[1, 25:] = 0
    with torch.no_grad():
        want = hf.encoder(input_ids=ids, attention_mask=mask).last_hidden_state
    got = OM.encoder_forward(sd, cfg, ids, mask)
    valid = mask.bool()
    assert torch.allclose(got[valid], want[valid], atol=2e-4, rtol=1e-4)
    assert torch.equal(got[~valid], torch.zeros_like(got[~valid]))


def test_decoder_logits_match_huggingface(tiny):
    hf, cfg, sd = tiny
    ids = torch.randint(0, 100, (2, 30), generator=torch.Generator().manual_seed(3))
    dec = torch.randint(0, 100, (2, 140), generator=torch.Generator().manual_seed(4))
    with torch.no_grad():
        want = hf(input_ids=ids, decoder_input_ids=dec).logits
    mem = OM.encoder_forward(sd, cfg, ids)
    got = OM.lm_logits(sd, cfg, OM.decoder_forward(sd, cfg, dec, mem))
    assert torch.allclose(got, want, atol=5e-4, rtol=1e-4)


def test_untied_gated_gelu_logits_match_huggingface():
    """T5 v1.1 / Flan layout: gated-gelu feed-forward, untied lm head, no rescale before the head."""
    from transformers import T5Config as HFConfig, T5ForConditionalGeneration
    torch.manual_seed(1)
    hf_cfg = HFConfig(vocab_size=100, d_model=32, d_kv=8, d_ff=64, num_layers=2, num_decoder_layers=2, num_heads=4,
                      relative_attention_num_buckets=32, relative_attention_max_distance=128, dropout_rate=0.0,
                      feed_forward_proj="gated-gelu", tie_word_embeddings=False, decoder_start_token_id=0)
    hf = T5ForConditionalGeneration(hf_cfg).eval()
    with torch.no_grad():
        for p in hf.parameters():
            p.copy_(torch.randn_like(p) * 0.3)
    cfg = T5Config(vocab_size=100, d_model=32, d_kv=8, d_ff=64, num_layers=2, num_heads=4, dropout_rate=0.0,
                   feed_forward_proj="gated-gelu", tie_word_embeddings=False)
    sd = {k: v.detach().clone() for k, v in hf.state_dict().items()}
    ids = torch.randint(0, 100, (2, 30), generator=torch.Generator().manual_seed(3))
    dec = torch.randint(0, 100, (2, 20), generator=torch.Generator().manual_seed(4))
    with torch.no_grad():
        want = hf(input_ids=ids, decoder_input_ids=dec).logits
    got = OM.lm_logits(sd, cfg, OM.decoder_forward(sd, cfg, dec, OM.encoder_forward(sd, cfg, ids)))
    assert torch.allclose(got, want, atol=5e-4, rtol=1e-4)
    # and the product's model class agrees with the oracle on the host-side bookkeeping: untied head, no rescale
    from turbot5_amd import T5Model
    m = T5Model(cfg)
    assert m.lm_head.weight is not m.shared.weight and m.lm_scale == 1.0
    tied = T5Model(cfg.copy(tie_word_embeddings=True))
    assert tied.lm_head.weight is tied.shared.weight and tied.lm_scale == 32 ** -0.5
