"""Timing of kvq_mla_prefill_attn at DeepSeek-V2 prefill shapes (128 heads, 128 + 64 / 128 dims, bf16): the
program behind profiles/mla_prefill_attn_h128.md.  Not collected by pytest (no test_ prefix); run it as
    python3 tests/perf_mla_prefill.py [--once]
It prints one line per shape: milliseconds per call and TFLOP/s over the visible (query, key) pairs."""
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "vllm-metax_amd"))
from vllm_metax_amd import _custom_ops as ops  # noqa: E402

SHAPES = (("context chunk: 4 x 2048 queries, 8192 keys each, unmasked", 4, 2048, 8192, False),
          ("new tokens: 4 x 2048 causal", 4, 2048, 2048, True),
          ("new tokens: 1 x 8192 causal", 1, 8192, 8192, True))


def main():
    once = "--once" in sys.argv
    dev = "cuda:0"
    H, nope, rope, dv = 128, 128, 64, 128
    for name, B, ql, kl, causal in SHAPES:
        T, S = B * ql, B * kl
        q = torch.randn(T, H, nope + rope, device=dev, dtype=torch.bfloat16)
        kv = torch.randn(S, H, nope + dv, device=dev, dtype=torch.bfloat16)
        kpe = torch.randn(S, rope, device=dev, dtype=torch.bfloat16)
        cuq = torch.arange(0, T + 1, ql, dtype=torch.int32, device=dev)
        cuk = torch.arange(0, S + 1, kl, dtype=torch.int32, device=dev)
        out = torch.empty(T, H, dv, device=dev, dtype=torch.bfloat16)
        lse = torch.empty(H, T, device=dev)

        def call():
            ops.mla_prefill_attention(q, kv[..., :nope], kpe, kv[..., nope:], cuq, cuk, ql, (nope + rope) ** -0.5,
                                      causal, out=out, lse=lse)

        n = 1 if once else 10
        for _ in range(0 if once else 3):
            call()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / n
        flops = B * ql * kl * (0.5 if causal else 1.0) * H * (nope + rope + dv) * 2
        print(f"{name}: {ms:.3f} ms, {flops / ms / 1e9:.1f} TFLOP/s", flush=True)


if __name__ == "__main__":
    main()
