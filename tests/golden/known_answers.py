"""Integer / boolean known answers held by the reference's own unit tests (data only).

Sources: tests/core/test_nn/test_attention_helpers.py:10-103 and
tests/transformer/test_data_utils.py:12-86 of the reference.
"""

# --- dense attention mask -------------------------------------------------------------------
MASK_CU_SEQLENS = [0, 2, 4, 6, 9, 12, 18]
MASK_SEQ_LEN = 6
# 1 = attention allowed (the function returns the inverse, True = masked), shape [3, 6, 6]
MASK_ALLOWED_CAUSAL = [
    [[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [0, 0, 1, 0, 0, 0],
     [0, 0, 1, 1, 0, 0], [0, 0, 0, 0, 1, 0], [0, 0, 0, 0, 1, 1]],
    [[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0],
     [0, 0, 0, 1, 0, 0], [0, 0, 0, 1, 1, 0], [0, 0, 0, 1, 1, 1]],
    [[1, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0],
     [1, 1, 1, 1, 0, 0], [1, 1, 1, 1, 1, 0], [1, 1, 1, 1, 1, 1]],
]
MASK_ALLOWED_BIDIRECTIONAL = [
    [[1, 1, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0], [0, 0, 1, 1, 0, 0],
     [0, 0, 1, 1, 0, 0], [0, 0, 0, 0, 1, 1], [0, 0, 0, 0, 1, 1]],
    [[1, 1, 1, 0, 0, 0], [1, 1, 1, 0, 0, 0], [1, 1, 1, 0, 0, 0],
     [0, 0, 0, 1, 1, 1], [0, 0, 0, 1, 1, 1], [0, 0, 0, 1, 1, 1]],
    [[1, 1, 1, 1, 1, 1]] * 6,
]
MASK_MAX_SEQ_LENGTH = 6

# --- cumulative sequence lengths / position ids ----------------------------------------------
TOKEN_IDS = [[1, 2, 3, 0, 1, 2], [1, 2, 3, 4, 5, 6], [1, 2, 3, 4, 5, 0]]
CU_WITH_RESET = [0, 4, 6, 12, 18]
CU_WITHOUT_RESET = [0, 6, 12, 18]
POSITION_IDS_WITH_RESET = [[0, 1, 2, 3, 0, 1], [0, 1, 2, 3, 4, 5], [0, 1, 2, 3, 4, 5]]
POSITION_IDS_WITHOUT_RESET = [[0, 1, 2, 3, 4, 5]] * 3
PADDING_INPUT = [0, 4, 8, 12]
PADDING_PAD_TO = 16
PADDING_EXPECTED = [0, 4, 8, 12] + [-1] * 12
