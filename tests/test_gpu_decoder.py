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


@pytest.mark.parametrize("heads,kv_heads,k_block", [(4, 4, 64), (4, 4, 256), (8, 2, 256)])
def test_decoder_step_replayed_from_a_graph_equals_the_eager_steps(heads, kv_heads, k_block):
    """The decoder step with the cache's lengths on the device is captured once and replayed per token.  Every replay is
    checked: its logits must equal those of the same steps launched eagerly on a twin cache, bit for bit (same kernels,
    same launch sizes), with the host's own work and synchronisations between the replays; the planes, rest buffers and
    lengths the two runs leave behind must be equal as well.  Crosses the 128- and 192-token flushes."""
    from alignedkv_amd.model.decoder_harness import DecoderConfig, RandomLlamaDecoder, make_cache
    cfg = DecoderConfig(num_hidden_layers=3, hidden_size=128 * heads, num_attention_heads=heads, num_key_value_heads=kv_heads,
                        intermediate_size=1024, vocab_size=2000, max_position_embeddings=512)
    model = RandomLlamaDecoder(cfg, seed=7)
    B, prefill, steps = 2, 100, 100
    prompt = torch.randint(0, cfg.vocab_size, (B, prefill), device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))
    eager = make_cache("alignedkv_device_lengths", cfg, B, 320, k_block=k_block)
    want_tokens, want_logits = model.generate(prompt, steps, eager)
    graphed = make_cache("alignedkv_graph", cfg, B, 320, k_block=k_block)
    tokens, logits = model.generate_graphed(prompt, steps, graphed, forced_tokens=want_tokens)
    for s in range(steps):
        assert torch.equal(logits[s], want_logits[s]), f"replay {s}: max |dlogit| {(logits[s] - want_logits[s]).abs().max().item()}"
    assert torch.equal(tokens, want_tokens)
    a, b = eager.inner, graphed.inner
    for layer in range(cfg.num_hidden_layers):
        assert a.seq_lens[layer].cpu().tolist() == [prefill + steps - 1] * B == b.seq_lens[layer].cpu().tolist()
        for x, y in zip(a.k_planes[layer] + a.v_planes[layer], b.k_planes[layer] + b.v_planes[layer]):
            assert torch.equal(x, y)
        n = (prefill + steps - 1) % 64
        assert torch.equal(a.restk[layer][:, :n], b.restk[layer][:, :n]) and torch.equal(a.restv[layer][:, :n], b.restv[layer][:, :n])
        assert torch.equal(a.k_colmax[layer], b.k_colmax[layer]) and torch.equal(a.v_colmax[layer], b.v_colmax[layer])
    # and against dense torch attention, as the other cache kinds above
    ref_tokens, ref_logits = model.generate(prompt, steps, make_cache("dense_torch", cfg, B, 320), forced_tokens=want_tokens)
    err = (logits - ref_logits).abs().max().item()
    assert err <= 6e-2 * max(1.0, ref_logits.abs().max().item()), f"max |dlogit| {err}"


def test_config5_full_size_decoder_with_alignedkv_cache():
    """The 32-layer Llama-2-7B-shaped decoder (d = 4096, 32 heads x 128, fp16 weights ~ N(0, 0.02)) at batch 8: a
    128-token prompt, then 256 greedy steps with the AlignedKV cache in every layer (the loop of the reference's
    model/KVCache_AlignedKV.py:92-135), teacher-forced with the tokens of the same decoder on dense torch attention.
    Layer 0's last step is replayed by the C restatement on the planes the run left behind."""
    import numpy as np
    from oracle import akv_oracle as O
    from tests.common import assert_step_output, oracle_decode_step_c
    from alignedkv_amd.model.decoder_harness import DecoderConfig, RandomLlamaDecoder, make_cache
    B, prefill, steps = 8, 128, 256
    max_len = prefill + steps + 64
    cfg = DecoderConfig(max_position_embeddings=max_len)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.head_dim) == (32, 4096, 32, 128)
    model = RandomLlamaDecoder(cfg, seed=5)
    prompt = torch.randint(0, cfg.vocab_size, (B, prefill), device="cuda", generator=torch.Generator(device="cuda").manual_seed(6))
    print("config 5: dense torch attention run", flush=True)
    ref_tokens, ref_logits = model.generate(prompt, steps, make_cache("dense_torch", cfg, B, max_len))
    cache = make_cache("alignedkv", cfg, B, max_len)
    assert cache.fused
    kc0, vc0 = cache.key_cache[0], cache.value_cache[0]
    kc0.record_levels = vc0.record_levels = True
    last = {}
    inner = cache.auto_compute

    def recording(q, k, v, layer_id, mask=None):
        out = inner(q, k, v, layer_id, mask)
        if layer_id == 0 and q.shape[1] == 1:
            last.update(q=q.clone(), k=k.clone(), v=v.clone(), out=out.clone(), probs=cache._probs.clone())
        return out

    cache.auto_compute = recording
    print("config 5: AlignedKV cache run", flush=True)
    tokens, logits = model.generate(prompt, steps, cache, forced_tokens=ref_tokens)
    n = prefill + steps - 1                      # tokens cached: the last greedy choice is not fed back
    for layer in range(cfg.num_hidden_layers):
        kc, vc = cache.key_cache[layer], cache.value_cache[layer]
        assert cache.get_seq_length(layer) == n
        assert kc.reststartpos == vc.reststartpos == n // 64 * 64 and kc.restklen == vc.restvlen == n % 64
    assert torch.isfinite(logits).all()
    err = (logits - ref_logits).abs().max().item()
    scale = ref_logits.abs().max().item()
    agree = (tokens == ref_tokens).float().mean().item()
    print(f"config 5: max |dlogit| {err:.4f} at logit scale {scale:.3f}, greedy agreement {agree * 100:.1f} %", flush=True)
    assert err <= 0.1 * max(1.0, scale), f"max |dlogit| {err} (logit scale {scale})"
    assert agree >= 0.6
    # layer 0, last step, against the C restatement: K levels and threshold bit exact, V levels bit exact for the
    # probabilities the kernels produced, output within 1e-3
    R, nrest = kc0.reststartpos, kc0.restklen
    host = lambda t: t.cpu().numpy()
    want, klv, vlv, amin, p = oracle_decode_step_c(
        [host(t) for t in (kc0.k_cache_first_8, kc0.k_cache_mid_4, kc0.k_cache_last_4)],
        [host(t) for t in (vc0.v_cache_first_8, vc0.v_cache_mid_4, vc0.v_cache_last_4)],
        host(kc0.k_cache_exp_column_max), host(vc0.v_cache_exp_column_max), host(last["q"]), host(last["k"]), host(last["v"]), R,
        rest_k=host(kc0.restk)[:, :nrest], rest_v=host(vc0.restv)[:, :nrest])
    assert np.array_equal(host(kc0.last_levels), klv), "K fetch levels differ"
    got_p = host(last["probs"])[:, :, :n]
    got_amin, got_vlv = host(vc0.last_alignment_min), host(vc0.last_levels)
    assert np.array_equal(got_vlv, O.v_levels(got_amin, O.as_bits(np.ascontiguousarray(got_p[:, :, :R]))))
    tv, ti = O.bucket_max(got_p[:, :, None, :R], n)
    ov = [host(t) for t in (vc0.v_cache_first_8,)]
    to = O.v_cache_test_compute(ov[0], O.as_bits(tv), ti)
    assert np.array_equal(got_amin, O.alignment_min(O.test_o_exponent(to), host(vc0.v_cache_exp_column_max)))
    assert (got_vlv != vlv).mean() <= 2e-3
    probs_equal = bool(np.array_equal(O.as_bits(np.ascontiguousarray(got_p)), O.as_bits(np.ascontiguousarray(p[:, :, 0, :n]))))
    assert_step_output(host(last["out"]), want, "config 5, layer 0, last step", probs_equal)
