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


def predictor_order_cases():
    """(name, weight_row, residual or None, expected bf16) with input = ones, for the code
    predictor's order (R17:12110-12124, 12622-12650): lane l takes the pairs k = 2l, 2l + 64, ...,
    first element of a pair first; an odd last column goes to lane 0 after its pairs; same tree."""
    cases = []

    def row(n, pairs):
        w = np.zeros(n, dtype=np.uint16)
        for k, v in pairs:
            w[k] = v
        return w

    # columns 0, 1 and 64 are one chain: 2^24 + 1 rounds back to 2^24, then -2^24 -> 0.
    # (the talker's order puts column 1 into another lane and gives 1)
    cases.append(("a_pair_and_the_pair_64_later_share_a_lane",
                  row(128, [(0, TWO24), (1, ONE), (64, NEG_TWO24)]), None, 0x0000))
    # inside a pair the first element is added first: 2^24, +1 (lost), +1 (lost), -2^24 -> 0.
    # (second element first: 1, +2^24 -> 2^24, -2^24 -> 0, +1 -> 1)
    cases.append(("first_element_of_a_pair_first",
                  row(128, [(0, TWO24), (1, ONE), (64, ONE), (65, NEG_TWO24)]), None, 0x0000))
    # column 2 belongs to lane 1, not to lane 0's chain: lane 0 cancels exactly, lane 1 keeps its 1.
    cases.append(("lanes_are_two_columns_apart",
                  row(128, [(0, TWO24), (2, ONE), (64, NEG_TWO24)]), None, ONE))
    # tree pairs lane l with l + 16 first: lanes 0 (column 0) and 16 (column 32) cancel, lane 8
    # (column 16) survives.  (a sequential sum over lanes would absorb the 1)
    cases.append(("tree_pairs_l_with_l_plus_16",
                  row(128, [(0, TWO24), (16, ONE), (32, NEG_TWO24)]), None, ONE))
    # residual joins after the rounding: bf16(1 + 2^-8 + 2^-9) = 1 + 2^-7; + 2^-8 is a tie -> 1 + 2^-6.
    cases.append(("residual_added_after_rounding",
                  row(128, [(0, ONE), (1, P2M8), (2, P2M9)]), P2M8, 0x3f82))
    # 67 columns: the pair (66, 67) does not exist, column 66 is added by lane 0 after its pairs:
    # lane 0 = 2^24 - 2^24 = 0, lane 1 keeps 0.5.  (lane 1 taking column 66 would lose its 0.5 to
    # -2^24 and the total would be 0)
    cases.append(("odd_last_column_goes_to_lane_0",
                  row(67, [(0, TWO24), (2, 0x3f00), (66, NEG_TWO24)]), None, 0x3f00))
    return cases
