"""Writes the committed fixtures under tests/golden/ from the CPU oracles (no reference import).

    python tests/golden/make_golden.py

logprob_cfg1_rows4.pt   first 4 token rows of the CPU-runnable configuration (bf16 [4,128,32000],
                        seed 0): logits, ids, fp32 and fp64 oracle outputs.
sampling_rows16.pt      16 bf16 rows of 4096 entries covering the edge cases (tie at the k-th value,
                        tie at the top-p cut, all-equal, single spike, k >= V, masked prefix, -inf
                        only, signed zeros), with uniforms, (T, top_k, top_p) cases and the ids of
                        both sampling oracles.
lmhead_extras.pt        hidden bf16 [40, 64] x W bf16 [500, 64] with ids: fp64 log-probabilities and entropies of the
                        fused lm_head operator; bf16 logits [6, 777] with ids and upstream gradients: the fp64 gradient
                        of the logprob operator (one row with a masked target); and the drawn token's log-probability
                        of the sampling rows above for the first sampling case.
Files hold tensors and plain Python scalars only; load them with torch.load(weights_only=True).
"""
import math
import sys
from pathlib import Path

import torch

HERE = Path(__file__).resolve().parent
REPO = HERE.parents[1]
for p in (REPO, REPO / "kernel-align_amd"):
    sys.path.insert(0, str(p))

from benchmarks.workloads import cfg1_logits  # noqa: E402
from oracle import exact, logprob_ref, sampling_ref  # noqa: E402

SAMPLING_CASES = [(0.7, 50, 0.9), (1.0, 50, None), (1.0, None, 0.9), (1.0, None, None), (1.3, 5, 0.5),
                  (0.7, 5000, 0.99)]


def sampling_rows():
    g = torch.Generator().manual_seed(99)
    rows = (torch.randn(16, 4096, generator=g) * 3.0).bfloat16()
    rows[0, :] = 2.0                                   # all equal
    rows[1, :] = 0.0
    rows[1, 1234] = 25.0                               # single spike
    rows[2] = ((rows[2].float() * 2).round() / 2).bfloat16()   # coarse grid: ties at k-th value and at the cut
    rows[3, :3000] = -math.inf                         # masked prefix
    rows[4, :] = -math.inf                             # -inf only (torch: NaN probabilities; here: uniform draw)
    rows[5, :] = 0.0
    rows[5, ::2] = -0.0                                # signed zeros
    rows[6, :60] = 9.0                                 # 60-way tie above everything else: cut lands inside it
    u = torch.rand(16, generator=g)
    u[7], u[8] = 0.0, 1 - 2.0 ** -24
    return rows, u


def main():
    logits, ids = cfg1_logits()
    l4, i4 = logits[0, :4].clone(), ids[0, :4].clone()
    torch.save({"logits": l4, "ids": i4, "logp_f32": logprob_ref.logprob_ref(l4, i4),
                "logp_f64": logprob_ref.logprob_f64(l4, i4)}, HERE / "logprob_cfg1_rows4.pt")
    rows, u = sampling_rows()
    blob = {"logits": rows, "uniforms": u, "cases": torch.tensor(
        [[t, k or 0, p if p is not None else 1.0] for t, k, p in SAMPLING_CASES], dtype=torch.float64)}
    for n, (t, k, p) in enumerate(SAMPLING_CASES):
        blob[f"ids_exact_{n}"] = exact.sample(rows, t, k, p, u)
        ref_ids, margin = sampling_ref.sample(rows, k, p, t, u)
        blob[f"ids_torch_{n}"] = ref_ids
        blob[f"margin_torch_{n}"] = margin
    torch.save(blob, HERE / "sampling_rows16.pt")
    g = torch.Generator().manual_seed(123)
    hidden = torch.randn(40, 64, generator=g).bfloat16()
    weight = (torch.randn(500, 64, generator=g) * 0.2).bfloat16()
    hid_ids = torch.randint(0, 500, (40,), generator=g)
    full = torch.nn.functional.linear(hidden.double(), weight.double())
    bl = (torch.randn(6, 777, generator=g) * 3).bfloat16()
    bi = torch.randint(0, 777, (6,), generator=g)
    bl[2, bi[2]] = -math.inf                             # a masked target: logp = -inf, finite gradient
    bg = torch.randn(6, generator=g)
    t0, k0, p0 = SAMPLING_CASES[0]
    _, drawn_lp = exact.sample_rows(rows, t0, k0, p0, u)
    torch.save({"hidden": hidden, "weight": weight, "ids": hid_ids,
                "logp_f64": logprob_ref.lmhead_logprob_ref(hidden, weight, hid_ids, dtype=torch.float64),
                "entropy_f64": logprob_ref.entropy_f64(full),
                "bwd_logits": bl, "bwd_ids": bi, "bwd_grad": bg,
                "bwd_dlogits_f64": logprob_ref.logprob_backward_closed_form(bl, bi, bg),
                "drawn_logprob_case0": drawn_lp}, HERE / "lmhead_extras.pt")
    print("wrote", sorted(p.name for p in HERE.glob("*.pt")))


if __name__ == "__main__":
    main()
