"""How far the engine may lie from the plain implementation, fixture by fixture.

The measure everywhere is ``max |engine - plain| / max |plain|`` over a request's logits. float32 runs are held
to 1e-4 (the reference accepts 1e-4 between its own ways of cutting, tests/model/test_qwen3_forward.cpp:84-86).
bfloat16 runs round every activation to 8 bits of mantissa, and how far that carries depends on the fixture's
widths and depth, so each fixture has a bound of its own: about three times the worst error seen over all its
traces with the kernels as they are (the figure beside each bound). A bound several times wider hid what it is
there to find: with 3e-2 for all, a page of tiny A's keys overwritten with another page's (1.3e-2) passed.
``test_a_corrupted_page_is_caught`` and its like hold each bound against such a fault.
"""

FLOAT32 = 1e-4

BFLOAT16 = {
    "tiny A": 1e-2,            # worst seen 3.7e-3 (the first tokens of a sequence)
    "tiny B": 2e-2,            # worst seen 7.3e-3 (decode steps, pages of 32 and 64)
    "serving widths": 2.5e-2,  # worst seen 9.8e-3 (row 256 of the 2100-token prompt; the streams 9.0e-3)
    "edge shapes": 1.5e-2,     # worst seen 5.0e-3 (three heads a group, head size 48)
    "run orders": 1.7e-2,      # worst seen 5.7e-3 (a window of 7 keys)
    "toy architecture": 1.2e-2,  # worst seen 3.7e-3
    "packed widths": 2e-2,     # worst seen ?
}

# float32 arithmetic over a narrower cache: the reference pins its own such pair (float32 activations over a
# float16 cache) at 3e-3 (tests/backend/test_paged_attention.cpp:70-103). Worst seen: 3.2e-4 over float16 pages,
# 2.4e-3 over bfloat16 ones, which keep three bits fewer.
NARROW_CACHE = {"float16": 1e-3, "bfloat16": 3e-3}
