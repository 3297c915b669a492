"""The parity bars for attention outputs, shared by the randomized GPU tests.

The stated bar is max-abs 2e-2 (16-bit) or 2e-5 (fp32) against the oracle.
Where few tokens are visible the outputs have magnitude 1 to 4, one bf16 step
there is up to 1.6e-2, and the oracle (which rounds scores, probabilities and
output to the element type as the reference does, attention.py:107-134) is
itself up to 2.3e-2 away from the float64 result.  So an output is also held
to the float64 result, with a tighter bar (relative above magnitude 1: the
kernels keep scores and the normalisation in fp32), and its distance to the
oracle may pass the stated bar only where the oracle's own distance to float64
explains it.

That second allowance is fenced: it exists for contexts of a few tokens only.
A case whose shortest visible context is 64 tokens or more (every shape inside
the benchmark configurations' ranges) is held to the stated bar alone, and
every use of the allowance is counted and reported at the end of the run."""
import torch

RELAX_BELOW_CTX = 64   # the allowance is refused from this visible context length on
TALLY = {"cases": 0, "relaxed_cases": 0, "relaxed_elements": 0}

ORACLE_BAR = {torch.bfloat16: 2e-2, torch.float16: 2e-2, torch.float32: 2e-5}
FLOAT64_BAR = {torch.bfloat16: 1e-2, torch.float16: 2e-3, torch.float32: 2e-5}


def hold(out, ref, truth, dtype, min_ctx, what=""):
    """out: the HIP path; ref: the oracle in the element type; truth: the oracle's arithmetic in
    float64; min_ctx: the fewest keys any query row of the case sees."""
    out, ref, truth = out.detach().cpu().double(), ref.double(), truth.double()
    TALLY["cases"] += 1
    assert torch.isfinite(out).all(), what
    bar64 = FLOAT64_BAR[dtype] * truth.abs().clamp(min=1.0)
    miss64 = ((out - truth).abs() - bar64).max().item()
    assert miss64 <= 0, f"{what} vs float64: {miss64} beyond the bar"
    diff = (out - ref).abs()
    if min_ctx >= RELAX_BELOW_CTX:
        assert diff.max().item() <= ORACLE_BAR[dtype], \
            f"{what} vs oracle: max|diff| {diff.max().item()} > {ORACLE_BAR[dtype]} (no allowance: contexts >= {min_ctx})"
        return
    allowed = torch.maximum(torch.full_like(truth, ORACLE_BAR[dtype]), (ref - truth).abs() + bar64)
    miss = (diff - allowed).max().item()
    assert miss <= 0, f"{what} vs oracle: {miss} beyond the bar; max|diff| {diff.max().item()}"
    used = int((diff > ORACLE_BAR[dtype]).sum())
    if used:
        TALLY["relaxed_cases"] += 1
        TALLY["relaxed_elements"] += used
        print(f"parity_bars: {used} of {diff.numel()} elements beyond {ORACLE_BAR[dtype]} against the oracle, "
              f"within the oracle's own distance to float64 (shortest context {min_ctx}) {what}", flush=True)
