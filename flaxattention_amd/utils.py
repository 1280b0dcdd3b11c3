"""Diagnostics with the surface of flaxattention/utils.py: the dense post-mod score (or mask) matrix of one
(batch, head) and a picture of it.  Not on the attention path: the matrix is evaluated with torch on whatever
device the tensors live on, exactly as the mods are written (scalar functions broadcast over index grids)."""
import math
from pathlib import Path
from typing import Optional

import torch

from .core.common import _mask_mod_signature, _score_mod_signature

Array = torch.Tensor


def create_score_mod(query: Array, key: Array, score_mod: Optional[_score_mod_signature],
                     mask_mod: Optional[_mask_mod_signature], scale: Optional[float] = None,
                     batch_idx: int = 0, head_idx: int = 0) -> Array:
    """`[1, 1, M, N]`: `score_mod(scale * q k^T, b, h, q_idx, kv_idx)` for `query [M, D]`, `key [N, D]`, or the
    boolean `mask_mod(b, h, q_idx, kv_idx)` when no score_mod is given (flaxattention/utils.py:17-49; as there a
    score_mod takes precedence over a mask_mod)."""
    M, N = query.shape[0], key.shape[0]
    dev = query.device
    b = torch.full((1, 1, 1, 1), batch_idx, dtype=torch.int32, device=dev)
    h = torch.full((1, 1, 1, 1), head_idx, dtype=torch.int32, device=dev)
    m = torch.arange(M, dtype=torch.int32, device=dev).view(1, 1, M, 1)
    n = torch.arange(N, dtype=torch.int32, device=dev).view(1, 1, 1, N)
    if score_mod is not None:
        scale_factor = 1.0 / math.sqrt(query.shape[-1]) if scale is None else scale
        scores = (query @ key.transpose(-1, -2)) * scale_factor
        out = score_mod(scores.view(1, 1, M, N), b, h, m, n)
    else:
        out = mask_mod(b, h, m, n)
    return torch.as_tensor(out, device=dev).expand(1, 1, M, N)


def _name_to_title(name: str) -> str:
    return name.replace("_", " ").title()


def _token_grid(ax, n_q: int, n_kv: int) -> None:
    """Per-token tick labels and cell borders; only drawn for matrices of at most 32 x 32."""
    import numpy as np
    ax.set_xticks(range(n_kv), labels=[f"KV{j}" for j in range(n_kv)], fontsize=16, rotation=45 if n_kv > 12 else 0)
    ax.set_yticks(range(n_q), labels=[f"Q{i}" for i in range(n_q)], fontsize=16)
    for axis, n in ((ax.xaxis, n_kv), (ax.yaxis, n_q)):
        axis.set_ticks(np.arange(n + 1) - 0.5, minor=True)
    ax.grid(which="minor", color="black", linestyle="-", linewidth=2)


def visualize_attention_scores(query: Array, key: Array, score_mod: Optional[_score_mod_signature] = None,
                               mask_mod: Optional[_mask_mod_signature] = None, device: str = "cuda",
                               name: str = "attention_scores", path: Optional[Path] = None, batch_idx: int = 0,
                               head_idx: int = 0, scale: Optional[float] = None) -> None:
    """Save a heat map of the post-mod scores (or of the mask) of one (batch, head) of `query` / `key`
    `[B, H, L, D]` as `<name>.png`, or at `path` with the suffix `.png`.  Arguments, title, axis labels, colour
    maps (viridis for scores, cividis for masks) and the tick rule follow flaxattention/utils.py:58-139;
    `device` is accepted for signature parity and unused, the tensors are used where they are."""
    if score_mod is None and mask_mod is None:
        raise AssertionError("Must provide either score_mod or mask_mod")
    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    grid = create_score_mod(query[batch_idx, head_idx], key[batch_idx, head_idx], score_mod=score_mod,
                            mask_mod=mask_mod, scale=scale, batch_idx=batch_idx, head_idx=head_idx)[0, 0]
    n_q, n_kv = grid.shape
    out = (Path(name) if path is None else Path(path)).with_suffix(".png")
    which = f"Batch {batch_idx}, Head {head_idx}" if (batch_idx, head_idx) != (0, 0) else ""

    fig, ax = plt.subplots(figsize=(12, 10))
    try:
        image = ax.imshow(grid.float().cpu().numpy(), aspect="auto", cmap="cividis" if score_mod is None else "viridis")
        fig.colorbar(image)
        ax.set_title(f"{_name_to_title(name)}\n{which}", fontsize=20)
        ax.set_xlabel("Key Tokens", fontsize=18)
        ax.set_ylabel("Query Tokens", fontsize=18)
        ax.tick_params(axis="x", top=True, labeltop=True, bottom=False, labelbottom=False)   # key axis on top
        if max(n_q, n_kv) <= 32:
            _token_grid(ax, n_q, n_kv)
        fig.tight_layout()
        fig.savefig(out, dpi=300, bbox_inches="tight")
    finally:
        plt.close(fig)
    print(f"Visualization saved as {out}")
