"""Slot order of the kernels' register unpack, mirrored from csrc/gptq_unpack.h (SLOT4 / SLOT3):
register r, half h of an unpacked lane block holds code ``CODE_OF_SLOT[2 r + h]``.  A host test
compiles the header and checks these tables against it."""

CODE_OF_SLOT4 = [0, 4, 1, 5, 2, 6, 3, 7]
CODE_OF_SLOT3 = [0, 6, 1, 7, 2, 8, 3, 9, 4, 10, 5, 11, 12, 18, 13, 19,
                 14, 20, 15, 21, 16, 22, 17, 23, 24, 30, 25, 31, 26, 28, 27, 29]


def code_of_slot(bits: int):
    return CODE_OF_SLOT4 if bits == 4 else CODE_OF_SLOT3


def slot_of_code(bits: int):
    table = code_of_slot(bits)
    inv = [0] * len(table)
    for slot, code in enumerate(table):
        inv[code] = slot
    return inv
