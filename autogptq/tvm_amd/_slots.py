"""Slot order of the kernels' register unpack, mirrored from csrc/gptq_unpack.h (SLOT4 / SLOT3 / SLOT8 /
SLOT2): register r, half h of an unpacked lane block holds code ``CODE_OF_SLOT[2 r + h]``.  A host test
compiles the header and checks these tables against it."""

CODE_OF_SLOT4 = [0, 4, 1, 5, 2, 6, 3, 7]
CODE_OF_SLOT3 = [0, 6, 1, 7, 2, 8, 3, 9, 4, 10, 5, 11, 12, 18, 13, 19,
                 14, 20, 15, 21, 16, 22, 17, 23, 24, 30, 25, 31, 26, 28, 27, 29]
CODE_OF_SLOT8 = [0, 2, 1, 3]
CODE_OF_SLOT2 = [0, 8, 1, 9, 2, 10, 3, 11, 4, 12, 5, 13, 6, 14, 7, 15]

_TABLES = {2: CODE_OF_SLOT2, 3: CODE_OF_SLOT3, 4: CODE_OF_SLOT4, 8: CODE_OF_SLOT8}

# The register unpack leaves (base + code) in each half register; the base of position e of an octet:
BASE_OF_POSITION = {
    2: [1024, 1024, 256, 256, 64, 64, 16, 16],
    3: [1024, 256, 128, 32, 1024, 256, 128, 32],
    4: [1024, 1024, 64, 64, 1024, 1024, 64, 64],
    8: [1024] * 8,
}


def code_of_slot(bits: int):
    """The table of one period of the width's permutation (4, 8, 16 or 32 codes)."""
    return _TABLES[bits]


def slot_of_code(bits: int):
    table = code_of_slot(bits)
    inv = [0] * len(table)
    for slot, code in enumerate(table):
        inv[code] = slot
    return inv


def lane_field_of_position(bits: int):
    """For the 32 codes of a lane of the tiled format: the stream field that holds position s."""
    table = code_of_slot(bits)
    n = len(table)
    return [(s // n) * n + table[s % n] for s in range(32)]
