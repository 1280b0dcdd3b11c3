"""The walk-through of flaxattention's examples/example.py on the MI355X engine: an ALiBi score_mod with a
causal sliding window of 10 on [8,8,2048,64] fp16, once through `flax_attention` with a block mask and once through
`flax_attention_pallas` with the mask_mod, the two compared to two decimals and timed over 10 calls; then the gradient
of the same call, and (with --pictures DIR) the four pictures the reference ships in visualizations/."""
import argparse
import sys
from pathlib import Path
from timeit import default_timer as timer

import numpy as np
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
from flaxattention_amd import and_masks, create_block_mask, flax_attention, flax_attention_pallas  # noqa: E402
from flaxattention_amd.masks import causal_mask, generate_attention_sink, generate_sliding_window  # noqa: E402
from flaxattention_amd.mods import generate_alibi_bias  # noqa: E402
from flaxattention_amd.utils import visualize_attention_scores  # noqa: E402


def timed(fn, n=10):
    fn()
    torch.cuda.synchronize()
    start = timer()
    for _ in range(n):
        fn()
    torch.cuda.synchronize()
    return timer() - start


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--pictures", default=None, help="directory for the visualisation PNGs (not drawn when omitted)")
    args = ap.parse_args()
    dev = torch.device("cuda", 0)
    batch_size, num_heads, seq_len_q, seq_len_kv, feature_size = 8, 8, 2048, 2048, 64

    def normal(seed, length):
        g = torch.Generator().manual_seed(seed)
        return torch.randn(batch_size, num_heads, length, feature_size, generator=g).to(torch.float16).to(dev)
    key, query, value = normal(0, seq_len_kv), normal(1, seq_len_q), normal(2, seq_len_kv)

    merged_mask = and_masks(causal_mask, generate_sliding_window(10))
    block_mask = create_block_mask(merged_mask, batch_size, num_heads, seq_len_q, seq_len_kv)
    print("Block mask:", block_mask)
    alibi = generate_alibi_bias(num_heads)

    output = flax_attention(query, key, value, score_mod=alibi, block_mask=block_mask)
    print("flax_attention, 10 calls:", timed(lambda: flax_attention(query, key, value, score_mod=alibi, block_mask=block_mask)), "s")
    print("Output shape:", tuple(output.shape))

    output_pallas = flax_attention_pallas(query, key, value, score_mod=alibi, mask_mod=merged_mask)
    print("Output Pallas shape:", tuple(output_pallas.shape))
    np.testing.assert_almost_equal(output.float().cpu().numpy(), output_pallas.float().cpu().numpy(), decimal=2)
    print("flax_attention and flax_attention_pallas agree to two decimals")
    print("flax_attention_pallas, 10 calls:",
          timed(lambda: flax_attention_pallas(query, key, value, score_mod=alibi, mask_mod=merged_mask)), "s")

    q, k, v = (t.clone().requires_grad_(True) for t in (query, key, value))

    def step():
        q.grad = k.grad = v.grad = None
        flax_attention(q, k, v, score_mod=alibi, block_mask=block_mask).sum().backward()
    print("forward + gradient, 10 calls:", timed(step), "s")
    print("Gradient shapes:", tuple(q.grad.shape), tuple(k.grad.shape), tuple(v.grad.shape))

    if args.pictures:
        out = Path(args.pictures)
        out.mkdir(parents=True, exist_ok=True)
        small_q, small_k = query[:, :, :16], key[:, :, :16]
        for name, kw in (("alibi_bias", dict(score_mod=alibi)), ("causal_mask", dict(mask_mod=causal_mask)),
                         ("sliding_window", dict(mask_mod=generate_sliding_window(4))),
                         ("attention_sink", dict(mask_mod=generate_attention_sink(4, 2)))):
            visualize_attention_scores(small_q, small_k, name=name, path=out / name, **kw)


if __name__ == "__main__":
    main()
