"""Hand-traced known-answer tiles for the reordering compressor.

Every expected stream below was worked out on paper from the TEXT of the
reference (csrc/SpMM_API.cu:132-156 helpers, :235-351 per-tile procedure),
not produced by running any implementation.  They pin the choices a
restatement can plausibly get wrong:

  bank      = (swizzled column / 2) % 32, swizzled column = n ^ ((m % 8) << 3)
  position  = m * 64 + swizzled column                         (:252-261)
  argmin / argmax take the LOWEST bank index on ties (strict < / >)  (:132-156)
  padding   = (4 - nnz % 4) % 4 items {value 0x0000, position = first zero
              position seen in scan order in the emptiest bank}      (:274-287)
  drain     = tail lanes first (v outer, lane inner), then main lanes
              (r, v, lane), each pop taking the BACK of the fullest bank (:306-325)
  write-out = main then tail, each lane popped from the BACK, so a lane's
              items come out in the reverse of the order it received them (:328-346)

A case is a dict: shape (M, K); "nz": {(m, n): fp16 bits} (global row / column);
"items": expected Compressed_A as (bits, local_m, local_n) triples or
("pad", local_m, local_n) for a padding item, in stream order;
"offsets": expected TileOffsets.
"""

ONE, TWO, THREE, FOUR = 0x3C00, 0x4000, 0x4200, 0x4400


def _v(m, n):
    """Distinct fp16 bit pattern per position used by the larger cases (all normal numbers)."""
    return 0x3C00 + (m // 8) * 64 + n


CASES = {}

# 1. Four nonzeros in four different banks, one vector (tail only, Rem = 1).
#    Row 0 has swizzle 0, so bank = n/2: n = 0,2,4,6 -> banks 0,1,2,3, all of size 1.
#    Tail fill for lane 0: argmax over equal sizes takes the lowest bank each time:
#    bank0, bank1, bank2, bank3.  The lane is written back to front: 3,2,1,0.
CASES["tail_distinct_banks"] = dict(
    shape=(128, 64),
    nz={(0, 0): ONE, (0, 2): TWO, (0, 4): THREE, (0, 6): FOUR},
    items=[(FOUR, 0, 6), (THREE, 0, 4), (TWO, 0, 2), (ONE, 0, 0)],
    offsets=[0, 1, 1],
)

# 2. Two banks with two items each: bank 0 = [A(0,0), B(0,1)], bank 5 = [C(0,10), D(0,11)].
#    Pops: tie 2/2 -> bank 0 back = B; then bank 5 (2 > 1) back = D; tie 1/1 -> bank 0: A; bank 5: C.
#    Lane 0 received [B, D, A, C]; emitted reversed: C, A, D, B.
CASES["tail_lifo_and_ties"] = dict(
    shape=(128, 64),
    nz={(0, 0): ONE, (0, 1): TWO, (0, 10): THREE, (0, 11): FOUR},
    items=[(THREE, 0, 10), (ONE, 0, 0), (FOUR, 0, 11), (TWO, 0, 1)],
    offsets=[0, 1, 1],
)

# 3. Three nonzeros (banks 0,1,2) -> one padding item.  Emptiest bank, lowest index: bank 3.
#    Bank 3 = swizzled columns 6,7; first zero seen in scan order is (0,6) -> position 6.
#    Then four single-item banks 0..3 as in case 1: emitted 3,2,1,0.
CASES["pad_one"] = dict(
    shape=(128, 64),
    nz={(0, 0): ONE, (0, 2): TWO, (0, 4): THREE},
    items=[("pad", 0, 6), (THREE, 0, 4), (TWO, 0, 2), (ONE, 0, 0)],
    offsets=[0, 1, 1],
)

# 4. One nonzero in bank 0 -> three padding items go to banks 1, 2, 3 in turn
#    (each time the lowest-index empty bank), at (0,2), (0,4), (0,6).
CASES["pad_three"] = dict(
    shape=(128, 64),
    nz={(0, 0): ONE},
    items=[("pad", 0, 6), ("pad", 0, 4), ("pad", 0, 2), (ONE, 0, 0)],
    offsets=[0, 1, 1],
)

# 5. Nothing to store.
CASES["all_zero"] = dict(shape=(128, 64), nz={}, items=[], offsets=[0, 0, 0])

# 6. Rows 0 and 8 full (swizzle 0 in both): bank b holds, in scan order,
#    i0=(0,2b) i1=(0,2b+1) i2=(8,2b) i3=(8,2b+1).  128 items = 32 vectors: main only (Rep 1, Rem 0).
#    Fill pass v: all banks are level, so lane l pops bank l's back: lane l receives [i3,i2,i1,i0].
#    Emitted reversed at out[l*4 + v]: i0,i1,i2,i3 of bank l.
_rows_0_8 = {(m, n): _v(m, n) for m in (0, 8) for n in range(64)}
CASES["main_level_banks"] = dict(
    shape=(128, 64),
    nz=dict(_rows_0_8),
    items=[(_v(m, n), m, n) for b in range(32) for (m, n) in ((0, 2 * b), (0, 2 * b + 1), (8, 2 * b), (8, 2 * b + 1))],
    offsets=[0, 32, 32],
)

# 7. Case 6 plus four more items in bank 0: (16,0) (16,1) (24,0) (24,1).  132 items = 33 vectors:
#    Rep 1, Rem 1.  The tail lane is filled FIRST: bank 0 is the fullest four times in a row and
#    gives (24,1) (24,0) (16,1) (16,0); the banks are then level and the main part is case 6.
#    The tail is written AFTER the main part, reversed: (16,0) (16,1) (24,0) (24,1).
_extra = [(16, 0), (16, 1), (24, 0), (24, 1)]
CASES["main_plus_tail"] = dict(
    shape=(128, 64),
    nz={**_rows_0_8, **{p: _v(*p) for p in _extra}},
    items=CASES["main_level_banks"]["items"] + [(_v(m, n), m, n) for (m, n) in _extra],
    offsets=[0, 33, 33],
)

# 8. Uneven banks, main only: case 6 without (8,2),(8,3) (bank 1 keeps c0=(0,2), c1=(0,3)) and with
#    (16,0),(16,1) added to bank 0 (a0..a5 = (0,0)(0,1)(8,0)(8,1)(16,0)(16,1)).  128 items.
#    Pass 0: lane0<-a5 (6 is max), lane1<-a4 (5), lane2<-a3 (tie at 4 -> bank 0), then bank 0 has 3 and
#            lanes 3..31 take the back (i3) of banks 2..30.  Bank 31 still has 4.
#    Pass 1: lane0<-i3 of bank 31 (the only 4); everything is 3 except bank 1 (2): lane1<-a2;
#            lanes 2..31 take i2 of banks 2..31.  Now every bank has 2.
#    Pass 2: lane l takes bank l: a1, c1, i1(l).   Pass 3: a0, c0, i0(l).
#    Emitted reversed per lane:
#      lane 0: a0 a1 i3(31) a5      lane 1: c0 c1 a2 a4      lane 2: i0 i1 i2 (bank 2), a3
#      lane l>=3: i0(l) i1(l) i2(l) i3(l-1)
def _i(b, j):
    return [(0, 2 * b), (0, 2 * b + 1), (8, 2 * b), (8, 2 * b + 1)][j]


_a = [(0, 0), (0, 1), (8, 0), (8, 1), (16, 0), (16, 1)]
_uneven_nz = {p: _v(*p) for p in _rows_0_8 if p not in ((8, 2), (8, 3))}
_uneven_nz.update({(16, 0): _v(16, 0), (16, 1): _v(16, 1)})
_uneven_order = [_a[0], _a[1], _i(31, 3), _a[5], (0, 2), (0, 3), _a[2], _a[4], _i(2, 0), _i(2, 1), _i(2, 2), _a[3]]
for _l in range(3, 32):
    _uneven_order += [_i(_l, 0), _i(_l, 1), _i(_l, 2), _i(_l - 1, 3)]
CASES["main_uneven_banks"] = dict(
    shape=(128, 64),
    nz=_uneven_nz,
    items=[(_v(m, n), m, n) for (m, n) in _uneven_order],
    offsets=[0, 32, 32],
)

# 9. What counts as zero: -0 (0x8000) and NaNs (0x7E00, 0xFE00) are dropped; a subnormal (0x0001),
#    +inf (0x7C00), -inf (0xFC00) and -1.0 (0xBC00) are kept: banks 2,3,4,6 -> emitted 6,4,3,2.
CASES["zero_test"] = dict(
    shape=(128, 64),
    nz={(0, 0): 0x8000, (0, 2): 0x7E00, (0, 4): 0x0001, (0, 6): 0x7C00, (0, 8): 0xFC00, (0, 10): 0xFE00, (0, 12): 0xBC00},
    items=[(0xBC00, 0, 12), (0xFC00, 0, 8), (0x7C00, 0, 6), (0x0001, 0, 4)],
    offsets=[0, 1, 1],
)

# 10. The swizzle: (1,0) -> col 0^8 = 8, bank 4; (3,5) -> 5^24 = 29, bank 14;
#     (127,63) -> 63^56 = 7, bank 3; (9,32) -> 32^8 = 40, bank 20.  Emitted in descending bank order.
CASES["swizzle"] = dict(
    shape=(128, 64),
    nz={(1, 0): ONE, (3, 5): TWO, (127, 63): THREE, (9, 32): FOUR},
    items=[(FOUR, 9, 32), (TWO, 3, 5), (ONE, 1, 0), (THREE, 127, 63)],
    offsets=[0, 1, 1],
    positions=[9 * 64 + 40, 3 * 64 + 29, 1 * 64 + 8, 127 * 64 + 7],
)

# 11. 2 x 2 tiles, row-major tile order: case 1 in tile (0,0), tile (0,1) empty,
#     case 3 in tile (1,0), case 2 in tile (1,1).
CASES["four_tiles"] = dict(
    shape=(256, 128),
    nz={(0, 0): ONE, (0, 2): TWO, (0, 4): THREE, (0, 6): FOUR,
        (128, 0): ONE, (128, 2): TWO, (128, 4): THREE,
        (128, 64): ONE, (128, 65): TWO, (128, 74): THREE, (128, 75): FOUR},
    items=[(FOUR, 0, 6), (THREE, 0, 4), (TWO, 0, 2), (ONE, 0, 0),
           ("pad", 0, 6), (THREE, 0, 4), (TWO, 0, 2), (ONE, 0, 0),
           (THREE, 0, 10), (ONE, 0, 0), (FOUR, 0, 11), (TWO, 0, 1)],
    offsets=[0, 1, 1, 2, 3, 3],
)

# No-reorder variant (csrc/SpMM_API.cu:439-474): scan order, and the first `pad` dropped
# elements met in scan order are emitted in place with their OWN bits.
# nnz = 3 -> pad 1: (0,0) = -0 is the first dropped element and is emitted as 0x8000 at position 0;
# the NaN at (0,2) comes after the padding is used up and is dropped.
NOREORDER_CASES = {
    "pad_keeps_bits": dict(
        shape=(128, 64),
        nz={(0, 0): 0x8000, (0, 1): ONE, (0, 2): 0x7E00, (0, 3): TWO, (0, 4): THREE},
        items=[(0x8000, 0, 0), (ONE, 0, 1), (TWO, 0, 3), (THREE, 0, 4)],
        offsets=[0, 1, 1],
    ),
    "scan_order": dict(
        shape=(128, 64),
        nz={(5, 7): FOUR, (0, 63): ONE, (0, 2): TWO, (127, 0): THREE},
        items=[(TWO, 0, 2), (ONE, 0, 63), (FOUR, 5, 7), (THREE, 127, 0)],
        offsets=[0, 1, 1],
    ),
}


def build_matrix(case):
    import numpy as np

    a = np.zeros(case["shape"], dtype=np.uint16)
    for (m, n), bits in case["nz"].items():
        a[m, n] = bits
    return a


def expected_stream(case):
    """Expected Compressed_A as uint32 values."""
    out = []
    for bits, m, n in case["items"]:
        pos = m * 64 + (n ^ ((m % 8) << 3))
        out.append(((0 if bits == "pad" else bits) | (pos << 16)) & 0xFFFFFFFF)
    return out
