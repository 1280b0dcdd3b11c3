"""Decode timing, the measurement flaxattention's examples/benchmark_decoding.py makes: one to a few
query rows against a long KV cache, through the dense-API entry point and through the split-KV
decode kernel, plus the q_len sweep that shows where the prefill kernel takes over (100 iterations
each, seconds for the 100)."""
import sys
from pathlib import Path
from timeit import default_timer as timer

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
from flaxattention_amd import create_block_mask, flax_attention  # noqa: E402
from flaxattention_amd.masks import offset_causal_mask  # noqa: E402


def checkerboard(score, batch, head, q_idx, k_idx):
    score = torch.where((k_idx - q_idx) % 2 == 0, score * 0.5, score)
    score = torch.where((k_idx - q_idx) % 2 == 1, score * 2.0, score)
    return score


def timed(fn, n=100):
    fn()
    torch.cuda.synchronize()
    start = timer()
    for _ in range(n):
        fn()
    torch.cuda.synchronize()
    return timer() - start


if __name__ == "__main__":
    dev = torch.device("cuda", 0)
    batch_size, num_heads, feature_size = 8, 8, 64
    for seq_len_kv in (2048, 16384):
        gen = lambda seed, L: torch.randn(batch_size, num_heads, L, feature_size, dtype=torch.float32,
                                          generator=torch.Generator().manual_seed(seed)).to(torch.float16).to(dev)
        key, value = gen(0, seq_len_kv), gen(2, seq_len_kv)
        for seq_len_q in (1, 16, 64, 128):
            query = gen(1, seq_len_q)
            bm = create_block_mask(offset_causal_mask(seq_len_kv - seq_len_q), batch_size, num_heads, seq_len_q, seq_len_kv, device=dev)
            t_auto = timed(lambda: flax_attention(query, key, value, score_mod=checkerboard, block_mask=bm))
            t_pre = timed(lambda: flax_attention(query, key, value, score_mod=checkerboard, block_mask=bm,
                                                 kernel_options={"decode": False}))
            line = f"KV {seq_len_kv:6d} q_len {seq_len_q:4d}: default path {t_auto:.4f} s, prefill kernel {t_pre:.4f} s"
            if seq_len_q <= 64:
                t_dec = timed(lambda: flax_attention(query, key, value, score_mod=checkerboard, block_mask=bm,
                                                     kernel_options={"decode": True}))
                line += f", split-KV decode kernel {t_dec:.4f} s"
            print(line, flush=True)
