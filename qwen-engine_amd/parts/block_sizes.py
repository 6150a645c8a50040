"""Sizes that the parts of a block agree on for steps of few rows (decode)."""

# Up to this many rows of a step, a part may be handed the stream, what is to be added to it and the
# norm instead of the normed rows: its first product then does the residual sum and the norm.
FEW_ROWS = 16
# ... and a branch's last product is then cut along K into at most this many partial products:
# every block of the product that adds them up reads all of them for all rows.
FEW_ROWS_PARTS = 4
# ... and only a product against a matrix of at most this many elements does the sum and the norm itself: a
# larger one is bound by the stream of its weights, which stands still while the prologue runs (at the
# 8B sizes a decode step of one request took 7 % longer with the prologue than with the norm's kernel).
FEW_ROWS_MAX_WEIGHT = 8 << 20
