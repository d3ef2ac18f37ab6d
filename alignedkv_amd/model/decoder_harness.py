"""Random-init Llama-shaped decoder that drives QuantizedCache_AlignedKV end to end.

The reference wires its cache into Hugging Face's Llama through model/Llama_AlignedKV.py (written
against transformers 4.44) and needs pretrained weights from the network.  This harness keeps the part
of that file which matters for the hot path -- q/k/v projections shaped [bsz, seq, heads, head_dim]
(not transposed), rotary embedding applied with that layout, `cache.auto_compute(q, k, v, layer, mask)`,
o_proj (model/Llama_AlignedKV.py:91-113,150-157) -- around a plain pre-norm SwiGLU decoder with fp16
weights drawn from N(0, 0.02), so that prefill + greedy decode run offline with the AlignedKV cache in
every layer.  Everything except the attention core is stock torch; it is a test vehicle, not a model zoo.

    python -m alignedkv_amd.model.decoder_harness --layers 32 --hidden 4096 --heads 32 --batch 8 \
        --prefill 128 --steps 256
"""
from __future__ import annotations

import argparse
import math
import time
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from .KVCache_AlignedKV import QuantizedCache_AlignedKV
from .ragged_gqa_cache import RaggedGQACache


@dataclass
class DecoderConfig:
    num_hidden_layers: int = 32
    hidden_size: int = 4096
    num_attention_heads: int = 32
    num_key_value_heads: int = 32
    intermediate_size: int = 11008
    vocab_size: int = 32000
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    max_position_embeddings: int = 4096

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    return (w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype))


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


class DenseTorchCache:
    """Dense fp16 K/V in torch with the semantics of the reference's fallback branch
    (model/Llama_AlignedKV.py:119-140): the comparison partner of the AlignedKV cache."""

    def __init__(self, n_layers: int):
        self.k = [None] * n_layers
        self.v = [None] * n_layers

    def get_seq_length(self, layer: int = 0) -> int:
        return 0 if self.k[layer] is None else self.k[layer].shape[2]

    def auto_compute(self, q, k, v, layer: int, mask=None):
        q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
        if self.k[layer] is not None:
            k = torch.cat([self.k[layer], k], dim=2)
            v = torch.cat([self.v[layer], v], dim=2)
        self.k[layer], self.v[layer] = k, v
        if k.shape[1] != q.shape[1]:     # grouped-query heads: repeat_kv
            k, v = (t.repeat_interleave(q.shape[1] // t.shape[1], dim=1) for t in (k, v))
        w = torch.matmul(q, k.transpose(2, 3)) / math.sqrt(q.shape[-1])
        if mask is not None:
            w = w + mask[:, :, :, :k.shape[-2]]
        w = F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
        return torch.matmul(w, v).transpose(1, 2).contiguous()


class DeviceLengthCache:
    """`auto_compute` over RaggedGQACache: the lengths live on the device and the step advances them itself, and the
    launches of a decode step are sized by the capacity, so every argument of a step is the same from step to step
    and a whole decoder step can be captured in a HIP graph (RandomLlamaDecoder.generate_graphed).  Prefill as the
    reference's (dense attention on the incoming tensors, planes written on the side, model/KVCache_AlignedKV.py:92-99)."""

    def __init__(self, cfg: "DecoderConfig", bsz: int, max_len: int, device="cuda", k_block: int = 64):
        self.inner = RaggedGQACache(cfg.num_hidden_layers, bsz, max_len, cfg.num_attention_heads, cfg.num_key_value_heads,
                                    cfg.head_dim, device, k_block=k_block)
        self.groups = cfg.num_attention_heads // cfg.num_key_value_heads
        self._host_len = [0] * cfg.num_hidden_layers     # what get_seq_length reports (eager callers)

    def get_seq_length(self, layer: int = 0) -> int:
        return self._host_len[layer]

    def device_positions(self) -> torch.Tensor:
        """[1] int32: the position of the next token, read from the lengths of layer 0 (before its step advances them)."""
        return self.inner.seq_lens[0][:1]

    def auto_compute(self, q, k, v, layer: int, mask=None):
        S = q.shape[1]
        if S > 1:
            assert self._host_len[layer] == 0, "prefill goes into an empty cache"
            for b in range(q.shape[0]):
                self.inner.prefill(layer, b, k[b:b + 1], v[b:b + 1])
            self._host_len[layer] = S
            kr, vr = (t.repeat_interleave(self.groups, dim=2) if self.groups > 1 else t for t in (k, v))
            w = torch.matmul(q.transpose(1, 2), kr.permute(0, 2, 3, 1)) / math.sqrt(q.shape[-1])
            if mask is not None:
                w = w + mask
            w = F.softmax(w.float(), dim=-1).type_as(q)
            return torch.matmul(w, vr.transpose(1, 2)).transpose(1, 2).contiguous()
        assert mask is None
        self._host_len[layer] += 1
        return self.inner.decode(layer, q, k, v, bound=self.inner.max_seq_len - 1)

    def snapshot(self):
        c = self.inner
        return [(c.seq_lens[i].clone(), c.k_colmax[i].clone(), c.v_colmax[i].clone()) for i in range(c.n_layers)], list(self._host_len)

    def restore(self, snap):
        """Takes back the steps since snapshot(), as long as none of them crossed a 64-token boundary (the token rows
        they appended to the rest buffers are written again by the steps that follow)."""
        c = self.inner
        for i, (n, kc, vc) in enumerate(snap[0]):
            c.seq_lens[i].copy_(n)
            c.k_colmax[i].copy_(kc)
            c.v_colmax[i].copy_(vc)
        self._host_len = list(snap[1])


class RandomLlamaDecoder(torch.nn.Module):
    def __init__(self, cfg: DecoderConfig, device="cuda", seed: int = 0, dtype=torch.half):
        super().__init__()
        self.cfg = cfg
        g = torch.Generator(device=device).manual_seed(seed)

        def w(*shape):
            return (torch.randn(shape, device=device, generator=g) * 0.02).to(dtype)

        d, h, kv, hd, ff = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.intermediate_size
        self.embed = w(cfg.vocab_size, d)
        self.layers = []
        for _ in range(cfg.num_hidden_layers):
            self.layers.append(dict(wq=w(h * hd, d), wk=w(kv * hd, d), wv=w(kv * hd, d), wo=w(d, h * hd),
                                    w_gate=w(ff, d), w_up=w(ff, d), w_down=w(d, ff),
                                    ln1=torch.ones(d, device=device, dtype=dtype),
                                    ln2=torch.ones(d, device=device, dtype=dtype)))
        self.norm = torch.ones(d, device=device, dtype=dtype)
        self.lm_head = w(cfg.vocab_size, d)
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, hd, 2, device=device).float() / hd))
        self.inv_freq = inv

    def rope(self, positions: torch.Tensor, dtype):
        """cos/sin [1, seq, 1, head_dim] for the [bsz, seq, heads, head_dim] layout (unsqueeze_dim=2)."""
        f = torch.outer(positions.float(), self.inv_freq)
        emb = torch.cat((f, f), dim=-1)
        return emb.cos().to(dtype)[None, :, None, :], emb.sin().to(dtype)[None, :, None, :]

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, cache, positions: torch.Tensor = None) -> torch.Tensor:
        """input_ids [bsz, seq]; returns logits of the last position [bsz, vocab] (fp32).  positions: [seq] device
        tensor of the tokens' positions (default: counted from the cache's length on the host)."""
        cfg = self.cfg
        B, S = input_ids.shape
        x = self.embed[input_ids]
        if positions is None:
            start = cache.get_seq_length(0)
            positions = torch.arange(start, start + S, device=x.device)
        cos, sin = self.rope(positions, x.dtype)
        mask = None
        if S > 1:
            mask = torch.full((S, S), float("-inf"), device=x.device, dtype=x.dtype).triu(1)[None, None]
        for li, L in enumerate(self.layers):
            hn = rms_norm(x, L["ln1"], cfg.rms_norm_eps)
            q = F.linear(hn, L["wq"]).view(B, S, cfg.num_attention_heads, cfg.head_dim)
            k = F.linear(hn, L["wk"]).view(B, S, cfg.num_key_value_heads, cfg.head_dim)
            v = F.linear(hn, L["wv"]).view(B, S, cfg.num_key_value_heads, cfg.head_dim)
            q = q * cos + rotate_half(q) * sin
            k = k * cos + rotate_half(k) * sin
            a = cache.auto_compute(q.contiguous(), k.contiguous(), v.contiguous(), li, mask)
            x = x + F.linear(a.reshape(B, S, -1), L["wo"])
            hn = rms_norm(x, L["ln2"], cfg.rms_norm_eps)
            x = x + F.linear(F.silu(F.linear(hn, L["w_gate"])) * F.linear(hn, L["w_up"]), L["w_down"])
        x = rms_norm(x[:, -1], self.norm, cfg.rms_norm_eps)
        return F.linear(x, self.lm_head).float()

    @torch.no_grad()
    def generate(self, prompt_ids: torch.Tensor, steps: int, cache, forced_tokens: torch.Tensor = None, timings: dict = None):
        """Prefill + `steps` greedy decode steps.  With forced_tokens [bsz, steps] the model is teacher-forced
        (the fed token is given, the greedy choice is still recorded).  Returns (tokens [bsz, steps],
        logits [steps, bsz, vocab]).  timings: filled with prefill_s (one synchronisation after the prefill)."""
        t0 = time.perf_counter()
        logits = self.forward(prompt_ids, cache)
        if timings is not None:
            torch.cuda.synchronize()
            timings["prefill_s"] = time.perf_counter() - t0
        toks, all_logits = [], []
        for s in range(steps):
            nxt = logits.argmax(-1)
            toks.append(nxt)
            all_logits.append(logits)
            if s + 1 == steps:
                break
            feed = nxt if forced_tokens is None else forced_tokens[:, s]
            logits = self.forward(feed[:, None], cache)
        return torch.stack(toks, dim=1), torch.stack(all_logits, dim=0)


    @torch.no_grad()
    def generate_graphed(self, prompt_ids: torch.Tensor, steps: int, cache: DeviceLengthCache,
                         forced_tokens: torch.Tensor = None, timings: dict = None):
        """generate() with the decoder step (embedding to logits, the cache's step in every layer) captured once in a HIP
        graph and replayed per token: the host pays one graph launch and the arg-max per step.  The token fed and the
        position are device tensors (the position is the cache's own length).  Needs prefill + steps to stay inside one
        64-token block for the warm-up step that is taken back (see DeviceLengthCache.restore) -- any prompt length whose
        remainder modulo 64 is not 63."""
        assert prompt_ids.shape[1] % 64 != 63
        t0 = time.perf_counter()
        logits = self.forward(prompt_ids, cache)
        torch.cuda.synchronize()
        if timings is not None:
            timings["prefill_s"] = time.perf_counter() - t0
        t0 = time.perf_counter()
        feed = torch.zeros((prompt_ids.shape[0], 1), dtype=torch.long, device=prompt_ids.device)
        snap = cache.snapshot()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):       # first use of every library on the capture's kind of stream, outside the capture
            self.forward(feed, cache, positions=cache.device_positions())
        torch.cuda.current_stream().wait_stream(side)
        cache.restore(snap)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step_logits = self.forward(feed, cache, positions=cache.device_positions())
        cache.restore(snap)                 # (the capture ran nothing; the host-side count moved)
        torch.cuda.synchronize()
        if timings is not None:
            timings["capture_s"] = time.perf_counter() - t0
        toks, all_logits = [], []
        for s in range(steps):
            nxt = logits.argmax(-1)
            toks.append(nxt)
            all_logits.append(logits)
            if s + 1 == steps:
                break
            feed.copy_((nxt if forced_tokens is None else forced_tokens[:, s])[:, None])
            graph.replay()
            cache._host_len = [n + 1 for n in cache._host_len]
            logits = step_logits.clone()
        return torch.stack(toks, dim=1), torch.stack(all_logits, dim=0)


def make_cache(kind: str, cfg: DecoderConfig, bsz: int, max_len: int, device="cuda", k_block: int = 64):
    """kind: 'alignedkv' (fused step), 'alignedkv_ops' (the reference's op sequence), 'alignedkv_reference'
    (every plane read), 'dense_torch', 'alignedkv_graph' / 'alignedkv_device_lengths' (the step with lengths on the
    device, replayed from a HIP graph / launched eagerly)."""
    if kind == "dense_torch":
        return DenseTorchCache(cfg.num_hidden_layers)
    if kind in ("alignedkv_graph", "alignedkv_device_lengths"):
        return DeviceLengthCache(cfg, bsz, max_len, device, k_block=k_block)
    c = QuantizedCache_AlignedKV(cfg, bsz, max_len, device, torch.half, k_block=k_block)
    c.reference = kind == "alignedkv_reference"
    if kind == "alignedkv_ops":
        c.fused = False
    return c


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--ffn", type=int, default=11008)
    ap.add_argument("--vocab", type=int, default=32000)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prefill", type=int, default=128)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--kinds", default="dense_torch,alignedkv_reference,alignedkv")
    ap.add_argument("--k-block", type=int, default=64, help="tokens per block of the K planes (64 or 256)")
    a = ap.parse_args()
    cfg = DecoderConfig(a.layers, a.hidden, a.heads, a.heads, a.ffn, a.vocab, max_position_embeddings=a.prefill + a.steps + 64)
    model = RandomLlamaDecoder(cfg)
    prompt = torch.randint(0, a.vocab, (a.batch, a.prefill), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    base_tokens = base_logits = None
    for kind in a.kinds.split(","):
        cache = make_cache(kind, cfg, a.batch, a.prefill + a.steps + 64, k_block=a.k_block)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        timings = {}
        if kind == "alignedkv_graph":
            toks, logits = model.generate_graphed(prompt, a.steps, cache, forced_tokens=base_tokens, timings=timings)
        else:
            toks, logits = model.generate(prompt, a.steps, cache, forced_tokens=base_tokens, timings=timings)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0 - timings.get("capture_s", 0.0)
        decode = dt - timings["prefill_s"]
        line = (f"{kind:20s} {dt:7.2f} s  {a.batch * a.steps / dt:8.1f} tok/s  (prefill {timings['prefill_s']:.2f} s; the "
                f"{a.steps - 1} decode steps alone {decode * 1e3 / (a.steps - 1):.2f} ms/step = {a.batch * (a.steps - 1) / decode:.1f} tok/s)")
        if "capture_s" in timings:
            line += f"  (+ {timings['capture_s']:.2f} s once for the warm-up step and the capture)"
        if base_tokens is None:
            base_tokens, base_logits = toks, logits
        else:
            agree = (toks == base_tokens).float().mean().item()
            err = (logits - base_logits).abs().max().item()
            line += f"  greedy agreement with {a.kinds.split(',')[0]} (teacher forced) {agree * 100:.2f} %  max |dlogit| {err:.4f}"
        print(line, flush=True)


if __name__ == "__main__":
    main()
