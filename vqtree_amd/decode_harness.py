"""Llama-shaped greedy decode loop over a VQ-coded key cache (counterpart of the reference's generation demo `gen.py`
and of the seqlen_q == 1 branch of its attention module, ops/attn_vq.py:176-223, which the reference leaves
unimplemented).

Every layer keeps, per (batch, head): the additive-quantiser codes of its keys `[B,H,cap,M] uint8` and the values
`[B,H,cap,D]`.  A step projects the new token, rotates q to the clamped ReRoPE position, encodes the new key greedily
against the layer's codebooks (residual, nearest codeword; HIP encoder), appends code and value, and attends over the
whole cache with the HIP decode kernel.  With `exact_window = W` the last W keys are kept exactly as well (rotated at
their true positions) and scored with the query at its true position; the coded and the exact part are merged by
log-sum-exp.  The linear layers are plain torch matmuls (weights ~ N(0, 0.02)): they are plumbing around
the attention path, which is what this harness measures.

    python -m vqtree_amd.decode_harness --layers 32 --context 65536 --batch 4 --steps 128
"""
import argparse
import json
import math
import time

import torch

from .ops.attn_vq import apply_rope, attn_vq_decode, attn_vq_decode_windowed, rope_tables, rotate_half
from .ops.mini_vq import RESIDUAL, encode_keys


def encode_residual(x, codebooks):
    """Greedy additive (residual) encoding on the HIP key encoder: x [B,H,T,D], codebooks [H,M,K,D] ->
    codes [B,H,T,M] uint8."""
    return encode_keys(x, codebooks, RESIDUAL)[0]


class VQDecodeModel:
    """Random-init Llama-2-shaped decoder (RMSNorm, rotary attention over a VQ key cache, SwiGLU MLP)."""

    def __init__(self, layers, hidden, heads, head_dim, ffn, vocab, n_codebooks, window, capacity, batch,
                 dtype=torch.bfloat16, device="cuda", seed=5, cb_std=0.35, exact_window=0):
        g = torch.Generator(device=device).manual_seed(seed)
        w = lambda *s: (torch.randn(*s, generator=g, device=device, dtype=torch.float32) * 0.02).to(dtype)
        self.L, self.hidden, self.H, self.D, self.M = layers, hidden, heads, head_dim, n_codebooks
        self.window, self.capacity, self.B = window, capacity, batch
        self.exact_window = exact_window  # 0: every key is scored through its codes; W > 0: the last W keys exactly
        self.dtype, self.device = dtype, device
        self.embed = w(vocab, hidden)
        self.lm_head = w(hidden, vocab)
        self.layers = []
        for _ in range(layers):
            self.layers.append(dict(
                wqkv=w(hidden, 3 * heads * head_dim), wo=w(heads * head_dim, hidden),
                w_gate_up=w(hidden, 2 * ffn), w_down=w(ffn, hidden),
                codebooks=(torch.randn(heads, n_codebooks, 256, head_dim, generator=g, device=device) * cb_std).to(dtype),
                codes=torch.empty(batch, heads, capacity, n_codebooks, dtype=torch.uint8, device=device),
                values=torch.empty(batch, heads, capacity, head_dim, dtype=dtype, device=device),
                # the most recent exact keys (rotated at their true positions): rows [kwin_len - w, kwin_len) of a
                # 2W-row buffer that is compacted when it fills up, so the window is always one contiguous slice
                kwin=(torch.empty(batch, heads, 2 * exact_window, head_dim, dtype=dtype, device=device)
                      if exact_window else None),
            ))
        self.length = 0
        self.kwin_len = 0
        self.cos, self.sin = rope_tables(head_dim, max(capacity, window + 2), dtype=dtype, device=device)
        # every far key is seen at the clamped position
        self.cos_w, self.sin_w = self.cos[window + 1].contiguous(), self.sin[window + 1].contiguous()

    def fill_random_context(self, n_tokens, seed=6):
        """Synthetic cache contents standing in for a prefill of n_tokens (random codes, V ~ N(0,1))."""
        g = torch.Generator(device=self.device).manual_seed(seed)
        for layer in self.layers:
            layer["codes"][:, :, :n_tokens] = torch.randint(0, 256, (self.B, self.H, n_tokens, self.M), generator=g,
                                                            device=self.device, dtype=torch.uint8)
            for b in range(self.B):
                layer["values"][b, :, :n_tokens] = torch.randn(self.H, n_tokens, self.D, generator=g,
                                                               device=self.device).to(self.dtype)
            if self.exact_window:
                w = min(self.exact_window, n_tokens)
                layer["kwin"][:, :, :w] = torch.randn(self.B, self.H, w, self.D, generator=g,
                                                      device=self.device).to(self.dtype)
        self.length = n_tokens
        self.kwin_len = min(self.exact_window, n_tokens)

    @staticmethod
    def _rms(x):
        return (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-5)).to(x.dtype)

    def _attend(self, layer, q_raw, n, attention, win_end):
        """Attention of the new token (cache rows [0, n] are filled).  Coded keys are scored with the query at the
        clamped position window + 1, exact window keys with the query at its true position n."""
        scale = 1.0 / math.sqrt(self.D)
        codes, values = layer["codes"][:, :, : n + 1], layer["values"][:, :, : n + 1]
        if not self.exact_window and attention is None:
            # the clamped rotation of the query happens inside the lookup-table kernel
            return attn_vq_decode(q_raw.unsqueeze(2), codes, layer["codebooks"], values, softmax_scale=scale,
                                  rope=(self.cos_w, self.sin_w))
        q_far = apply_rope(q_raw.unsqueeze(2), self.cos, self.sin, self.window + 1)  # [B,H,1,D], one launch
        if not self.exact_window:
            return attention(q_far, codes, layer["codebooks"], values, softmax_scale=scale)
        w = min(self.exact_window, n + 1)
        k_win = layer["kwin"][:, :, win_end - w: win_end]
        q_win = (q_raw * self.cos[n] + rotate_half(q_raw) * self.sin[n]).unsqueeze(2)
        if attention is not None:
            return attention(q_far, q_win, codes, layer["codebooks"], values, k_win, softmax_scale=scale)
        return attn_vq_decode_windowed(q_far, codes, layer["codebooks"], values, k_win, softmax_scale=scale,
                                       q_window=q_win)

    def step(self, tokens, attention=None, return_logits=False, events=None):
        """One greedy decode step for token ids [B]; returns next token ids [B] (and the logits).  `attention`
        overrides the attention operator (tests pass a dense reference)."""
        B, H, D = self.B, self.H, self.D
        n = self.length
        if self.exact_window and self.kwin_len == 2 * self.exact_window:  # compact the window buffer
            for layer in self.layers:
                layer["kwin"][:, :, : self.exact_window] = layer["kwin"][:, :, self.exact_window:].clone()
            self.kwin_len = self.exact_window
        x = self.embed[tokens]  # [B, hidden]
        for layer in self.layers:
            h = self._rms(x)
            qkv = (h @ layer["wqkv"]).view(B, 3, H, D)
            q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]  # [B,H,D]
            layer["codes"][:, :, n] = encode_residual(k.unsqueeze(2), layer["codebooks"])[:, :, 0]
            layer["values"][:, :, n] = v
            if self.exact_window:
                layer["kwin"][:, :, self.kwin_len] = k * self.cos[n] + rotate_half(k) * self.sin[n]
            if events is not None:
                events.append(torch.cuda.Event(enable_timing=True))
                events[-1].record()
            o = self._attend(layer, q, n, attention, self.kwin_len + 1)
            if events is not None:
                events.append(torch.cuda.Event(enable_timing=True))
                events[-1].record()
            x = x + o.reshape(B, H * D) @ layer["wo"]
            h = self._rms(x)
            gate, up = (h @ layer["w_gate_up"]).chunk(2, dim=-1)
            x = x + (torch.nn.functional.silu(gate) * up) @ layer["w_down"]
        self.length = n + 1
        self.kwin_len += 1 if self.exact_window else 0
        logits = self._rms(x) @ self.lm_head
        return (logits.argmax(-1), logits) if return_logits else logits.argmax(-1)

    # ---------------------------------------------------------------------------------------------------------
    # the same step with every position-dependent quantity in device memory, so that it can be recorded once as a
    # HIP graph and replayed: cache writes by index_copy_ at `pos_dev`, attention over `n_dev` keys of the full
    # buffers, the next token kept in a static buffer
    # ---------------------------------------------------------------------------------------------------------
    def _init_device_state(self, tokens):
        from . import _lib

        assert not self.exact_window, "the recorded step codes every key"
        dev = self.device
        self.tok = tokens.clone()
        self.pos_dev = torch.tensor([self.length], dtype=torch.int64, device=dev)
        self.n_dev = torch.tensor([self.length + 1], dtype=torch.int32, device=dev)
        lib = _lib.load()
        self.splits = lib.vqa_decode_default_splits(self.B, self.H, self.capacity)
        self.ws = torch.empty(lib.vqa_decode_workspace_bytes(self.B, self.H, self.capacity, self.D, self.M, 256,
                                                             self.splits), dtype=torch.uint8, device=dev)
        self.attn_out = torch.empty(self.B, self.H, 1, self.D, dtype=self.dtype, device=dev)
        self.logits = None

    def _device_step(self):
        B, H, D = self.B, self.H, self.D
        x = self.embed[self.tok]
        for layer in self.layers:
            h = self._rms(x)
            qkv = (h @ layer["wqkv"]).view(B, 3, H, D)
            q, k, v = qkv[:, 0], qkv[:, 1], qkv[:, 2]
            layer["codes"].index_copy_(2, self.pos_dev, encode_residual(k.unsqueeze(2), layer["codebooks"]))
            layer["values"].index_copy_(2, self.pos_dev, v.unsqueeze(2))
            attn_vq_decode(q.unsqueeze(2), layer["codes"], layer["codebooks"], layer["values"],
                           softmax_scale=1.0 / math.sqrt(D), num_splits=self.splits, n_keys=self.n_dev,
                           out=self.attn_out, workspace=self.ws, rope=(self.cos_w, self.sin_w))
            x = x + self.attn_out.reshape(B, H * D) @ layer["wo"]
            h = self._rms(x)
            gate, up = (h @ layer["w_gate_up"]).chunk(2, dim=-1)
            x = x + (torch.nn.functional.silu(gate) * up) @ layer["w_down"]
        logits = self._rms(x) @ self.lm_head
        self.tok.copy_(logits.argmax(-1))
        self.pos_dev += 1
        self.n_dev += 1
        return logits

    def record_step(self, tokens):
        """Record one decode step as a HIP graph (after one warm-up step on a side stream, which already advances the
        cache by one token).  `replay_step()` then runs a step per call; `self.tok` holds the newest tokens and
        `self.logits` the logits of the last replayed step."""
        self._init_device_state(tokens)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._device_step()
        torch.cuda.current_stream().wait_stream(side)
        self.length += 1
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = self._device_step()
        return self

    def replay_step(self):
        self.graph.replay()
        self.length += 1
        return self.tok

    def attention_bytes_per_step(self):
        """Algorithmic bytes of the attention path per token step: per layer codes of the coded keys + V + exact
        window keys + codebooks + q/out."""
        e = 2
        n = self.length
        w = min(self.exact_window, n)
        per_layer = self.B * self.H * (n - w) * self.M + e * self.B * self.H * n * self.D \
            + e * self.B * self.H * w * self.D + e * self.H * self.M * 256 * self.D + 2 * e * self.B * self.H * self.D
        return self.L * per_layer


def run(layers=32, hidden=4096, heads=32, head_dim=128, ffn=11008, vocab=32000, n_codebooks=4, context=65536, batch=4,
        steps=128, warmup=4, window=1024, exact_window=0, graph=0, device="cuda"):
    model = VQDecodeModel(layers, hidden, heads, head_dim, ffn, vocab, n_codebooks, window,
                          context + steps + warmup + 10, batch, device=device, exact_window=exact_window)
    model.fill_random_context(context)
    g = torch.Generator(device=device).manual_seed(7)
    tokens = torch.randint(0, vocab, (batch,), generator=g, device=device)
    if graph:
        with torch.no_grad():
            model.record_step(tokens)
            for _ in range(warmup):
                model.replay_step()
            torch.cuda.synchronize()
            bytes_mid = None
            t0 = time.perf_counter()
            for s in range(steps):
                if s == steps // 2:
                    bytes_mid = model.attention_bytes_per_step()
                model.replay_step()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        return {
            "workload": f"{layers}-layer Llama-2-7B-shaped greedy decode, batch {batch}, context {context}, VQ key "
                        f"cache {n_codebooks}x256 per layer, {steps} steps, one HIP graph replay per step",
            "us_per_step": round(dt / steps * 1e6, 1),
            "attention_bytes_per_step": bytes_mid,
            "note": "whole-step wall time; the step (projections, MLP, key encoder, cache append, attention) is "
                    "recorded once with the cache position and key count in device memory",
        }
    with torch.no_grad():
        for _ in range(warmup):
            tokens = model.step(tokens)
        torch.cuda.synchronize()
        bytes_mid = None
        paced = []
        t0 = time.perf_counter()
        for s in range(steps):
            if s == steps // 2:
                bytes_mid = model.attention_bytes_per_step()
            tokens = model.step(tokens, events=paced)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        # The Python loop above is host-bound (about a thousand launches per step), so the GPU runs dry between the
        # launches of an attention call and the event intervals around the calls contain those gaps.  A second pass
        # measures the GPU time of the same calls with the host ahead of the GPU: every step starts with a device-side
        # sleep long enough for the host to queue the whole step behind it.
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        torch.cuda._sleep(10_000_000)
        b.record()
        b.synchronize()
        cycles_per_ms = 10_000_000 / a.elapsed_time(b)
        ahead_steps = min(steps, 8)
        events = []
        for s in range(ahead_steps):
            if s == ahead_steps // 2:
                bytes_mid = model.attention_bytes_per_step()
            torch.cuda._sleep(int(1.5 * dt / steps * 1e3 * cycles_per_ms))
            tokens = model.step(tokens, events=events)
            torch.cuda.synchronize()
    paced_us = sum(paced[i].elapsed_time(paced[i + 1]) for i in range(0, len(paced), 2)) / steps * 1e3
    steps_wall, steps = steps, ahead_steps
    us = dt / steps_wall * 1e6
    attn_us = sum(events[i].elapsed_time(events[i + 1]) for i in range(0, len(events), 2)) / steps * 1e3
    return {
        "workload": f"{layers}-layer Llama-2-7B-shaped greedy decode, batch {batch}, context {context}, VQ key cache "
                    f"{n_codebooks}x256 per layer, " + (f"last {exact_window} keys exact, " if exact_window else "")
                    + f"{steps_wall} steps",
        "us_per_step": round(us, 1),
        "attention_us_per_step": round(attn_us, 1),
        "attention_bytes_per_step": bytes_mid,
        "attention_GBps": round(bytes_mid / (attn_us * 1e-6) / 1e9, 1),
        "attention_hbm_frac": round(bytes_mid / (attn_us * 1e-6) / 8e12, 4),
        "attention_us_per_step_host_paced": round(paced_us, 1),
        "note": "us_per_step is whole-step wall time of the plain Python loop (projections, MLP, key encoder, "
                "attention), which is host-bound; attention_us_per_step sums HIP-event intervals around the attention "
                "calls of all layers (lookup table with the clamped rotary of the query, streaming kernel, merge) over "
                f"{ahead_steps} steps whose launches were queued ahead of the GPU behind a device-side sleep, i.e. GPU "
                "time without launch gaps; attention_us_per_step_host_paced is the same sum taken in the plain loop",
    }


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    for name, default in (("layers", 32), ("context", 65536), ("batch", 4), ("steps", 128), ("warmup", 4),
                          ("exact_window", 0), ("graph", 0)):
        ap.add_argument("--" + name, type=int, default=default)
    print(json.dumps(run(**vars(ap.parse_args()))))
