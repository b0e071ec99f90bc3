"""Bit widths of the packed int32 encodings shared by planner, dispatch and
tests; same values as reference moonep/constants.py:6-10 so that the shape
limits (R <= 128, K <= 32, NvS < 2**24) are the reference's."""

RANK_BITS = 7
KIDX_BITS = 7
