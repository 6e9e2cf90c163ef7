"""Writes tests/golden/find_blocks_golden.pt: input/output vectors of the
reference's own ``find_blocks_chunked`` (xattn/src/utils.py:44-191).

Run once, in the build container, where the reference checkout is mounted at
/root/reference:  ``python tests/golden/make_find_blocks_golden.py``.
Only ``xattn/src/utils.py`` is loaded (by file path; it imports nothing but
torch and its ``find_blocks_chunked`` is device-agnostic).  The committed
fixture holds data only: seeded inputs, arguments and the boolean masks the
reference returned on CPU.
"""
import importlib.util
import os

import torch

REF = "/root/reference/xattn/src/utils.py"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "find_blocks_golden.pt")


def causal_like(gen, heads, rows, cols, current_index, zero_future=True):
    """Block sums shaped like the estimator's: positive, future blocks zero."""
    x = torch.rand((1, heads, rows, cols), generator=gen, dtype=torch.float32) ** 3
    x[..., 0] += 0.5 * torch.rand((1, heads, rows), generator=gen)
    if zero_future:
        for r in range(rows):
            x[:, :, r, current_index + r + 1 :] = 0
    return x


def main():
    spec = importlib.util.spec_from_file_location("ref_utils", REF)
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)
    gen = torch.Generator().manual_seed(20240917)
    cases = []

    def add(name, x, current_index, threshold, causal):
        y = ref.find_blocks_chunked(
            x.clone(), current_index, threshold, None, decoding=False, mode="prefill", causal=causal
        )
        cases.append(
            dict(
                name=name,
                x=x,
                current_index=current_index,
                threshold=threshold if isinstance(threshold, torch.Tensor) else torch.tensor(threshold, dtype=torch.float64),
                threshold_is_tensor=isinstance(threshold, torch.Tensor),
                causal=causal,
                mask=y,
            )
        )

    for tau in (0.0, 0.3, 0.5, 0.9, 0.95, 1.0):
        add(f"causal_first_chunk_tau{tau}", causal_like(gen, 3, 8, 8, 0), 0, tau, True)
        add(f"causal_second_chunk_tau{tau}", causal_like(gen, 3, 8, 16, 8), 8, tau, True)
        add(f"causal_kv_offset_tau{tau}", causal_like(gen, 2, 4, 24, 20), 20, tau, True)
        add(f"noncausal_tau{tau}", torch.rand((1, 3, 6, 12), generator=gen) ** 2, 0, tau, False)
    per_head = torch.tensor([0.0, 0.9, 0.45, 1.0], dtype=torch.float32)
    add("causal_per_head", causal_like(gen, 4, 8, 16, 8), 8, per_head, True)
    add("noncausal_per_head", torch.rand((1, 4, 5, 9), generator=gen), 0, per_head, False)
    # dense (no zeroed future) causal input: exercises the tail clearing
    add("causal_dense_future", causal_like(gen, 2, 4, 16, 4, zero_future=False), 4, 0.9, True)
    # bf16-rounded sums, as the operator hands them over
    add(
        "causal_bf16_sums",
        causal_like(gen, 3, 8, 16, 8).to(torch.bfloat16),
        8,
        0.9,
        True,
    )
    torch.save(cases, OUT)
    print(f"wrote {len(cases)} cases to {OUT}")


if __name__ == "__main__":
    main()
