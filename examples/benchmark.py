"""Forward / gradient timing of flax_attention and flax_attention_pallas on [8,8,2048,64] fp16
with a checkerboard score_mod written as a plain Python function, the measurement
flaxattention's examples/benchmark.py makes (100 iterations each, seconds for the 100).
torch's scaled_dot_product_attention stands in for jax.nn.dot_product_attention as the
"no score_mod" comparison."""
import sys
from pathlib import Path
from timeit import default_timer as timer

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
from flaxattention_amd import create_block_mask, flax_attention, flax_attention_pallas  # noqa: E402


def checkerboard(score, batch, head, q_idx, k_idx):
    score = torch.where((k_idx - q_idx) % 2 == 0, score * 0.5, score)
    score = torch.where((k_idx - q_idx) % 2 == 1, score * 2.0, score)
    return score


def causal(batch, head, q_idx, k_idx):
    return q_idx >= k_idx


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
    batch_size, num_heads, seq_len_q, seq_len_kv, feature_size = 8, 8, 2048, 2048, 64
    gen = lambda seed, L: torch.randn(batch_size, num_heads, L, feature_size, dtype=torch.float32,
                                      generator=torch.Generator().manual_seed(seed)).to(torch.float16).to(dev)
    key, query, value = gen(0, seq_len_kv), gen(1, seq_len_q), gen(2, seq_len_kv)
    block_mask = create_block_mask(causal, batch_size, num_heads, seq_len_q, seq_len_kv, device=dev)

    print("flax_attention time taken:", timed(lambda: flax_attention(query, key, value, score_mod=checkerboard)))
    print("flax_attention (causal block mask) time taken:",
          timed(lambda: flax_attention(query, key, value, score_mod=checkerboard, block_mask=block_mask)))

    q_grad = query.clone().requires_grad_(True)

    def grad0():
        q_grad.grad = None
        flax_attention(q_grad, key, value, score_mod=checkerboard).sum().backward()
    print("flax_attention gradient time taken:", timed(grad0))

    print("flax_attention_pallas time taken:", timed(lambda: flax_attention_pallas(query, key, value, score_mod=checkerboard)))

    def grad1():
        q_grad.grad = None
        flax_attention_pallas(q_grad, key, value, score_mod=checkerboard).sum().backward()
    print("flax_attention_pallas gradient time taken:", timed(grad1))

    sdpa = torch.nn.functional.scaled_dot_product_attention
    print("torch scaled_dot_product_attention time taken (no score_mod):", timed(lambda: sdpa(query, key, value)))

    def grad2():
        q_grad.grad = None
        sdpa(q_grad, key, value).sum().backward()
    print("torch scaled_dot_product_attention gradient time taken (no score_mod):", timed(grad2))
