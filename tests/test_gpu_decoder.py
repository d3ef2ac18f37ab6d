"""End-to-end: a random-init Llama-shaped decoder (prefill + greedy decode, AlignedKV cache in every layer)
against the same decoder with dense torch attention, teacher-forced with the dense run's tokens."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind,tol", [("alignedkv_reference", 2e-2), ("alignedkv", 6e-2), ("alignedkv_ops", 6e-2)])
def test_decoder_with_alignedkv_cache_tracks_dense_attention(kind, tol):
    from alignedkv_amd.model.decoder_harness import DecoderConfig, RandomLlamaDecoder, make_cache
    cfg = DecoderConfig(num_hidden_layers=3, hidden_size=512, num_attention_heads=4, num_key_value_heads=4,
                        intermediate_size=1024, vocab_size=2000, max_position_embeddings=512)
    model = RandomLlamaDecoder(cfg, seed=3)
    B, prefill, steps = 2, 100, 80           # crosses the 128-token and 192-token flush boundaries
    prompt = torch.randint(0, cfg.vocab_size, (B, prefill), device="cuda", generator=torch.Generator(device="cuda").manual_seed(4))
    ref_tokens, ref_logits = model.generate(prompt, steps, make_cache("dense_torch", cfg, B, 256))
    cache = make_cache(kind, cfg, B, 256)
    tokens, logits = model.generate(prompt, steps, cache, forced_tokens=ref_tokens)
    assert cache.get_seq_length(0) == prefill + steps - 1
    assert cache.key_cache[2].reststartpos == (prefill + steps - 1) // 64 * 64
    assert torch.isfinite(logits).all()
    err = (logits - ref_logits).abs().max().item()
    scale = ref_logits.abs().max().item()
    assert err <= tol * max(1.0, scale), f"max |dlogit| {err} (logit scale {scale})"
    # random-init logits are nearly flat, so a greedy arg-max flips on tiny perturbations: the logit error
    # above is the criterion, token agreement only a sanity bound
    assert (tokens == ref_tokens).float().mean().item() >= (0.9 if kind == "alignedkv_reference" else 0.6)
