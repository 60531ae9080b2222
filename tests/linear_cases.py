"""Hand-built M = 1 linear cases whose bf16 result depends on the reference's evaluation order
(R17:15239-15266): 32 lane-strided fmaf chains in increasing k, the shfl_down tree 16/8/4/2/1,
bias added in fp32 before the rounding, residual added to the rounded value.  Shared by the
oracle pins (CPU) and the GPU parity tests."""
import numpy as np

ONE, TWO24, NEG_TWO24 = 0x3f80, 0x4b80, 0xcb80          # 1.0, 2^24, -2^24 as bf16
P2M8, P2M9, P2M10 = 0x3b80, 0x3b00, 0x3a80              # 2^-8, 2^-9, 2^-10
P15_2M9 = 0x3b40                                         # 1.5 * 2^-9 = 2^-9 + 2^-10


def order_cases():
    """(name, weight_row[96], bias or None, residual or None, expected bf16) with input = ones."""
    cases = []

    def row(pairs):
        w = np.zeros(96, dtype=np.uint16)
        for k, v in pairs:
            w[k] = v
        return w

    # one chain, increasing k: (2^24 + 1) rounds back to 2^24 before -2^24 arrives -> 0.
    # (adding -2^24 before the 1 would give 1)
    cases.append(("chain_order_increasing_k", row([(0, TWO24), (32, ONE), (64, NEG_TWO24)]), None, None, 0x0000))
    # chains are lane-strided: k = 0 and k = 32 share lane 0 (cancel exactly), k = 1 is lane 1 -> 1.
    # (contiguous chunks per lane would absorb the 1 into 2^24 and give 0)
    cases.append(("chains_are_lane_strided", row([(0, TWO24), (1, ONE), (32, NEG_TWO24)]), None, None, ONE))
    # tree pairs lane l with l+16 first: lanes 0 and 16 cancel, lane 8 survives -> 1.
    # (a sequential sum over lanes would absorb lane 8's 1 and give 0)
    cases.append(("tree_pairs_l_with_l_plus_16", row([(0, TWO24), (8, ONE), (16, NEG_TWO24)]), None, None, ONE))
    # bias joins in fp32 before the rounding: (1 + 2^-9 + 2^-10) + 1.5*2^-9 = 1 + 2^-8 + 2^-9 -> 1 + 2^-7.
    # (rounding first would give 1.0)
    cases.append(("bias_added_before_rounding", row([(0, ONE), (1, P2M9), (2, P2M10)]), P15_2M9, None, 0x3f81))
    # residual joins after the rounding: bf16(1 + 2^-8 + 2^-9) = 1 + 2^-7; + 2^-8 is a tie -> even -> 1 + 2^-6.
    # (a single rounding of the fp32 sum would give 1 + 2^-7)
    cases.append(("residual_added_after_rounding", row([(0, ONE), (1, P2M8), (2, P2M9)]), None, P2M8, 0x3f82))
    return cases
