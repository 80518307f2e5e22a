"""The numbers by which the parts and the kernels' faces choose between forms of a kernel.

They were measured on LFM2-sized layers (widths of 1024 to 4096) on one MI355X and decide speed
only: every form gives the same result for the shapes it takes.  They live here, not in the
parts, so that a part holds no size of any particular model; the C side of a step gets the same
numbers in its model description.
"""

# A projection whose consumer can add partial sums asks for them only above this many rows:
# 6144 x 2048 plus the conv step takes 13.0 us unsplit and 13.3 us in two K ranges at 8 rows, 18 us
# and 12 us at 64 rows.
PARTIAL_SUMS_MIN_ROWS = 16
# ... and in steps of up to this many rows whatever their segments (short prompt portions): with
# few rows the products of in_proj and qkv have too few blocks to fill the chip unless K is cut
# (in_proj of 128 rows: 9-12 us in four ranges against 22 us whole; the float partial sums of
# 512 rows would already cost more than the cut saves).  Above it only steps of single rows
# (decode at large batches) hand on partial sums.
PARTIAL_SUMS_MAX_ROWS = 256


def takes_partial_sums(rows: int, single_rows: bool) -> bool:
    """Whether in_proj / qkv of a step of ``rows`` rows hand their consumer partial sums."""
    return rows > PARTIAL_SUMS_MIN_ROWS and (rows <= PARTIAL_SUMS_MAX_ROWS or single_rows)

# Every bfloat16 matrix whose shape allows it (rows a multiple of 16, columns of 32) is kept in
# the order in which the product kernels load it (``ops.fragment_order``), and only so: decode
# steps stream it 10-20 % faster than rows (a step at batch 8: about a tenth), the block kernels
# of prompt steps as fast as rows, and the matrices' memory is needed once.  False keeps the
# matrices as the checkpoint has them.
FRAGMENT_ORDER = True

# The norm kernel hands its rows on in fragment order from this many rows on (up to 16): a step of
# the 1.2B shape takes 1.06 against 1.08 ms at 16 rows, 0.994 against 1.000 at 12, even at 8; with
# fewer rows the ordinary order is as fast or faster.
FRAGMENT_ROWS = True
FRAGMENT_ROWS_MIN = 8

# The conv layer's fused decode kernel (in_proj, gates, FIR, state shift in one) gives one block 16
# channels (8 below a width of 4096, where 16 would leave CUs without a block).  From
# FUSED_STEP_MIN_WIDTH on it beats the separate product (which may split K) plus the small step
# kernel for any number of rows up to 64; between FUSED_STEP_NARROW_WIDTH and it only up to
# FUSED_STEP_NARROW_ROWS rows (at a width of 2048, W in fragment order: 8.3 against 9.9 us for one
# row; 11.0 against 11.1 at 8 rows, 11.5 against 12.8 at 16; at a width of 1024 the separate
# kernels win).
FUSED_STEP_MIN_WIDTH = 4096
FUSED_STEP_NARROW_WIDTH = 2048
FUSED_STEP_NARROW_ROWS = 16

# A decode step's attention kernel normalises and rotates q and the row's own key itself and
# stores key and value (head sizes 64 and 128, rotate-half over the whole head, a projection that
# comes as bfloat16 rows, more than 512 keys) for steps of up to FUSED_QK_MAX_ROWS rows: every
# wave of the kernel does that work again, which a few hundred waves do faster than a kernel of
# its own would (a step of the 1.2B shape: 10 us less at 1 to 4 rows) and a thousand or more do
# not (7 us more at 6 rows, 12 at 8, 40 at 12).  0 switches it off.
FUSED_QK = True
FUSED_QK_MAX_ROWS = 4

# In a step that holds prompt portions, a single decoded token is one tile for the tiled attention
# kernel, and the block that gets it walks all its keys alone: 0.9 ms at 32 k keys, however short
# the portions beside it are.  From this many keys on such rows go to the decode kernel (keys
# split over blocks) instead: a second kernel and its merge (25-30 us a layer for up to 63 rows)
# against that walk.  16 requests with 32 k-token prompts: prompt steps 19 -> 14 ms.  With up to
# 63 rows of at most 2300 keys beside portions of 512 rows the two kernels took 49 us a layer where
# the tiled kernel alone took 43, hence not from 1024 on.
LONE_ROWS_FROM = 4096
