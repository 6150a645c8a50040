"""Sizes that the parts of a block agree on for steps of few rows (decode)."""

# Up to this many rows of a step, a part may be handed the stream, what is to be added to it and the
# norm instead of the normed rows: its first product then does the residual sum and the norm.
FEW_ROWS = 16
# ... and a branch's last product is then cut along K into at most this many partial products:
# every block of the product that adds them up reads all of them for all rows.
FEW_ROWS_PARTS = 4
