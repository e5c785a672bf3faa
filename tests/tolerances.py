"""Tolerances of the GPU parity tests.

fp32: every comparison with the CPU oracle uses rtol 1e-4 / atol 1e-5, from single ops to the whole
networks after 50 accumulated steps.

bf16 against the SAME bf16-rounded operands (op level): two bf16 ulps (rtol 2^-7).

bf16 networks against the fp32 oracle: rtol 2e-2 plus an absolute term derived from the output's scale.
Every layer rounds its delta (or, in a refresh, its activation) to bf16 once, a relative error of at most
u = 2^-8 per element; reservoirs and accumulation stay fp32.  Through the contracting non-linearities of
these networks (sigmoid / tanh heads, ReLU) the roundings of the ~16 layers on a path do not add up
linearly: measured on E2Depth-incr the deviation of a step's output is 1.1 - 1.7 u of its largest value, of
the accumulated sigmoid prediction 1.2 u, of EVFlowNet-incr's flow maps 1.3 - 2.4 u.  The tests allow
`roundoffs` (default 3) such units of the reference's scale, max|ref|, instead of a fixed absolute number.
One case needs more: a single step's flow DELTA of EVFlowNet-incr at the coarse scales, a 1x1 conv over
hundreds of channels of rounded deltas ten times its own size (cancellation): 2 - 12 u measured, 16 allowed.
"""
FP32_RTOL, FP32_ATOL = 1e-4, 1e-5
BF16_RTOL = 2e-2
BF16_U = 2.0 ** -8


def bf16_atol(ref, roundoffs: float = 3.0) -> float:
    """roundoffs * 2^-8 * max|ref| (a floor of 1e-3 on the scale keeps an all-zero reference testable)."""
    return roundoffs * BF16_U * max(float(ref.abs().max()), 1e-3)
