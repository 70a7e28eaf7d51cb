"""Compile every device-side text for gfx950, without a device.

The library compiles kernels at run time through the code-object manager
(libamd_comgr); this script asks the
freshly built library for representative kernel texts (flat and strided
elementwise variants, every reduction operation) and runs each through the
same compile the library uses.  It is the "does the device code
build" check of the build step.
"""
import ctypes as C
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(os.path.dirname(HERE), "libgpuarray.so")


class ElemwiseArg(C.Structure):
    _fields_ = [("name", C.c_char_p), ("typecode", C.c_int), ("flags", C.c_int)]


def main():
    lib = C.CDLL(LIB)
    lib.gpuarray_get_extension.restype = C.c_void_p
    lib.gpuarray_get_extension.argtypes = [C.c_char_p]

    def ext(name, res, args):
        return C.CFUNCTYPE(res, *args)(lib.gpuarray_get_extension(name))

    gen_e = ext(b"hip_elemwise_source", C.c_void_p,
                [C.c_char_p, C.c_char_p, C.c_uint, C.POINTER(ElemwiseArg), C.c_int, C.c_int,
                 C.c_uint, C.c_int, C.c_uint])
    gen_r = ext(b"hip_reduction_source", C.c_void_p,
                [C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint, C.c_uint, C.c_uint])
    gen_m = ext(b"hip_mapreduce_source", C.c_void_p,
                [C.c_int, C.c_char_p, C.c_char_p, C.c_int, C.c_char_p, C.c_char_p, C.c_uint,
                 C.POINTER(ElemwiseArg), C.c_int, C.c_uint, C.c_uint, C.c_uint, C.c_uint])
    comp = ext(b"hip_compile_only", C.c_int,
               [C.c_uint, C.POINTER(C.c_char_p), C.POINTER(C.c_size_t), C.POINTER(C.c_char_p)])

    def check(label, ptr):
        if not ptr:
            raise SystemExit("%s: generator failed" % label)
        arr = (C.c_char_p * 1)(C.string_at(ptr))
        log = C.c_char_p()
        if comp(1, arr, None, C.byref(log)) != 0:
            raise SystemExit("%s: does not compile for gfx950:\n%s" % (label, (log.value or b"").decode()))

    GA_FLOAT, GA_HALF, GA_INT, GA_LONG, GA_UBYTE, GA_BOOL, GA_DOUBLE = 11, 23, 5, 7, 2, 0, 12
    WROWS = 1 << 27      # the wave-per-row kernel in place of the general row kernel
    args = (ElemwiseArg * 3)(ElemwiseArg(b"a", GA_FLOAT, 2), ElemwiseArg(b"b", GA_FLOAT, 2),
                             ElemwiseArg(b"c", GA_FLOAT, 4))
    check("elemwise flat", gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 0, 0, 0, 0))
    for nd, idx64, tmask in [(1, 0, 0), (2, 0, 0), (3, 1, 0), (2, 0, 1), (3, 1, 3)]:
        check("elemwise strided nd=%d idx64=%d tmask=%x" % (nd, idx64, tmask),
              gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 1, nd, idx64, tmask))
    # four elements per lane: plain (umask in bits 16..) and transposed
    check("elemwise strided vec4 plain", gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 2, 2, 0, 0b101 << 16))
    check("elemwise strided vec4 transposed", gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 2, 3, 1, 0b001 | (0b110 << 16)))
    check("elemwise strided vec4 plain, streaming", gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 3, 2, 0, 0b101 << 16))
    GA_DOUBLE_ = 12
    dargs = (ElemwiseArg * 3)(ElemwiseArg(b"a", GA_DOUBLE_, 2), ElemwiseArg(b"b", GA_FLOAT, 2),
                              ElemwiseArg(b"c", GA_DOUBLE_, 4))
    check("elemwise strided, two doubles per lane", gen_e(b"", b"c = a*b + 0.5", 3, dargs, 0, 10, 2, 0, 0b101 << 16))
    check("elemwise strided vec4 transposed, streaming", gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 3, 3, 1, 0b001 | (0b110 << 16)))
    check("elemwise strided vec4 transposed, 128-tiles", gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 4, 3, 1, 0b001 | (0b110 << 16)))
    check("elemwise strided vec4 transposed, 128-tiles, windows on the result's 64-byte blocks",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 11, 3, 1, 0b001 | (0b110 << 16)))
    check("elemwise strided vec4 transposed, 128-tiles, windows on the result's 64-byte blocks, 32-bit offsets",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 11, 2, 0, 0b001 | (0b110 << 16)))
    check("elemwise strided vec4 transposed, 128-tiles, four-byte elements on any layout",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 12, 3, 1, 0b001 | (0b110 << 16)))
    check("elemwise strided vec4 transposed, 128-tiles, four-byte elements on any layout, 32-bit offsets",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 12, 2, 0, 0b001 | (0b100 << 16)))
    check("elemwise strided vec4 plain, four-byte elements on any layout",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 13, 2, 0, 0b101 << 16))
    check("elemwise strided vec4 plain, four-byte elements on any layout, 64-bit offsets, one operand element by element",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 13, 3, 1, 0b100 << 16))
    check("elemwise strided vec4 transposed, 8-byte elements (quads as two pairs)",
          gen_e(b"", b"c = a*b + 0.5", 3, dargs, 0, 3, 3, 1, 0b001 | (0b110 << 16)))
    check("elemwise strided vec4, 8-byte result written through a transposed tile",
          gen_e(b"", b"c = a*b + 0.5", 3, dargs, 0, 3, 2, 0, 0b100 | (0b011 << 16)))
    check("elemwise strided vec4 transposed, 128-tiles, operand constant along x",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 7, 2, 0, 0b001 | (0b100 << 16)))
    check("elemwise strided vec4 transposed, 128-tiles, operands constant along y",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 8, 2, 0, 0b001 | (0b110 << 16)))
    check("elemwise strided vec4 plain, operand constant along x",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 7, 2, 0, 0b100 << 16))
    check("elemwise flat, one operand read through the flat index's coordinates, 2 dims",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 9, 2, 0, 0b010))
    check("elemwise flat, one operand read a chunk at a time through the flat index's coordinates",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 9, 2, 0b010, 0b010))
    check("elemwise flat, an operand's chunks inside one row fetched with one load on four-byte boundaries",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 9, 2, 0b010 << 16, 0b010))
    check("elemwise flat, the same for two operands, 3 dims",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 9, 3, 0b011 << 16, 0b011))
    check("elemwise flat, two operands read through the flat index's coordinates, 3 dims",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 9, 3, 0, 0b011))
    # narrow planes in registers: short extent in nd, the short dim in bit 1 of idx64, streaming in bit 2
    check("elemwise narrow plane of 3 in registers: one operand with the short dim innermost, the rest chunked",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 14, 3, 0b100, 0b001 | (0b110 << 16)))
    check("elemwise narrow plane of 11 in registers: the result with the short dim innermost, 64-bit offsets",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 14, 11, 0b011, 0b100 | (0b001 << 16)))
    check("elemwise narrow plane of 8 in registers: operand through the LDS, result chunked on four-byte boundaries",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 14, 8, 0b11100, 0b001 | (0b110 << 16)))
    check("elemwise narrow plane of 5 in registers: the result through the LDS, 64-bit offsets",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 14, 5, 0b01011, 0b100 | (0b011 << 16)))
    check("elemwise narrow planes of 3 in registers, three dims: operand direct, result chunked",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 14, 3 | 256, 0b00100, 0b001 | (0b110 << 16)))
    check("elemwise narrow planes of 3 in registers, three dims: the result through the LDS",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 14, 3 | 256, 0b11110, 0b100 | (0b011 << 16)))
    check("elemwise narrow plane of 33 through the LDS: operand staged, result chunked",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 15, 33, 0b00100, 0b001 | (0b110 << 16)))
    check("elemwise narrow planes of 20 through the LDS, three dims: the result staged, chunks on four-byte boundaries",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 15, 20 | 256, 0b10111, 0b100 | (0b011 << 16)))
    check("elemwise narrow plane of 3 doubles in registers: the result through the LDS",
          gen_e(b"", b"c = a + c", 2, (ElemwiseArg * 2)(ElemwiseArg(b"a", GA_DOUBLE, 2), ElemwiseArg(b"c", GA_DOUBLE, 6)),
                0, 14, 3, 0b01110, 0b10 | (0b01 << 16)))
    check("elemwise narrow plane of 7 halves in registers, computed in floats",
          gen_e(b"", b"c = a + 1", 2, (ElemwiseArg * 2)(ElemwiseArg(b"a", GA_HALF, 2), ElemwiseArg(b"c", GA_HALF, 4)),
                2, 14, 7, 0b00100, 0b01 | (0b10 << 16)))
    check("elemwise narrow plane of 3 in registers: bytes with the short dim innermost to floats in planes",
          gen_e(b"", b"c = a * 0.5f", 2, (ElemwiseArg * 2)(ElemwiseArg(b"a", GA_UBYTE, 2), ElemwiseArg(b"c", GA_FLOAT, 4)),
                0, 14, 3, 0b10100, 0b01 | (0b10 << 16)))
    check("elemwise narrow plane of 3 in registers: floats in planes to bytes with the short dim innermost, staged",
          gen_e(b"", b"c = a", 2, (ElemwiseArg * 2)(ElemwiseArg(b"a", GA_FLOAT, 2), ElemwiseArg(b"c", GA_UBYTE, 4)),
                0, 14, 3, 0b01110, 0b10 | (0b01 << 16)))
    check("elemwise narrow plane of 4 in registers: bytes in planes to floats with the short dim innermost, staged",
          gen_e(b"", b"c = a", 2, (ElemwiseArg * 2)(ElemwiseArg(b"a", GA_UBYTE, 2), ElemwiseArg(b"c", GA_FLOAT, 4)),
                0, 14, 4, 0b01110, 0b10 | (0b01 << 16)))
    check("elemwise narrow planes of 3 in registers, three dims: a per-channel operand fetched once per channel",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 14, 3 | 256, 0b101100, 0b001 | (0b100 << 16)))
    check("elemwise tiles of records of 3: one operand's records along Y, the other's and the result's along X",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 16, 3, 0b100, 0b001 | (0b110 << 16)))
    check("elemwise tiles of records of 20, four dims, 64-bit offsets, one operand element by element",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 16, 20 | 256, 0b001, 0b001 | (0b100 << 16)))
    check("elemwise tiles of records of 3, windows moved onto the result's 64-byte blocks",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 16, 3, 0b1100, 0b001 | (0b110 << 16)))
    check("elemwise tiles of records of 50, four dims, 64-bit offsets, moved windows",
          gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 16, 50 | 256, 0b1001, 0b001 | (0b100 << 16)))
    bargs = (ElemwiseArg * 2)(ElemwiseArg(b"a", GA_UBYTE, 2), ElemwiseArg(b"c", GA_UBYTE, 4))
    check("elemwise tiles of records of 3 bytes, moved windows, tiles numbered along Y first",
          gen_e(b"", b"c = a", 2, bargs, 0, 16, 3, 0b11100, 0b01 | (0b10 << 16)))
    dargs2 = (ElemwiseArg * 2)(ElemwiseArg(b"a", GA_DOUBLE, 2), ElemwiseArg(b"c", GA_DOUBLE, 4))
    check("elemwise tiles of records of 2 doubles", gen_e(b"", b"c = a", 2, dargs2, 0, 16, 2, 0b0100, 0b01 | (0b10 << 16)))
    iargs = (ElemwiseArg * 2)(ElemwiseArg(b"a", GA_FLOAT, 2), ElemwiseArg(b"c", GA_FLOAT, 6))
    check("elemwise narrow plane of 4 in registers: an array read and written through the LDS",
          gen_e(b"", b"c = a + c", 2, iargs, 0, 14, 4, 0b01000, 0b10 | (0b01 << 16)))
    check("elemwise flat, 2 adjacent chunks per lane", gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 5, 0, 0, 0))
    check("elemwise flat, 4 adjacent chunks per lane", gen_e(b"", b"c = a*b + 0.5f", 3, args, 0, 6, 0, 0, 0))
    hargs = (ElemwiseArg * 2)(ElemwiseArg(b"src", GA_HALF, 2), ElemwiseArg(b"dst", GA_DOUBLE, 4))
    check("elemwise half->double copy", gen_e(b"", b"dst = src", 2, hargs, 2, 0, 0, 0, 0))
    n = 0
    for op in range(14):
        for src, d0 in [(GA_FLOAT, GA_FLOAT), (GA_INT, GA_LONG if op < 3 else GA_INT),
                        (GA_HALF, GA_FLOAT if op < 3 else GA_HALF)]:
            if op in (9, 10, 11) and src != GA_INT:
                continue          # bitwise ops: integers only
            if op in (12, 13):
                d0 = GA_BOOL
            check("reduction op=%d src=%d" % (op, src), gen_r(op, src, d0, GA_LONG, 256, 4, 4))
            n += 1
    check("reduction 64 lanes per output, general row kernel", gen_r(8, GA_FLOAT, GA_FLOAT, GA_LONG, 64, 4, 4))
    check("reduction wave-per-row", gen_r(8, GA_FLOAT, GA_FLOAT, GA_LONG, 64, 4, 4 | WROWS))
    for op, src in ((0, GA_FLOAT), (8, GA_FLOAT), (13, GA_UBYTE)):
        check("reduction with 32-bit divisions, op %d" % op,
              gen_r(op, src, GA_BOOL if op == 13 else GA_FLOAT, GA_LONG, 256, 4 if src == GA_FLOAT else 16, 4 | (1 << 28)))
        n += 1
    check("reduction bytes", gen_r(13, GA_UBYTE, GA_BOOL, GA_LONG, 64, 16, 1))
    check("reduction bytes, wave-per-row", gen_r(13, GA_UBYTE, GA_BOOL, GA_LONG, 64, 16, 1 | WROWS))
    # element step 2 inside a load (a [::2] view): 8 used of 16 fetched bytes
    check("reduction stepped bytes", gen_r(13, GA_UBYTE, GA_BOOL, GA_LONG, 64, 8 | (2 << 8), 1 | WROWS))
    check("reduction stepped halves", gen_r(0, GA_HALF, GA_FLOAT, GA_LONG, 256, 4 | (2 << 8), 1))
    check("reduction short rows in batches of 4", gen_r(13, GA_UBYTE, GA_BOOL, GA_LONG, 64, 8 | (2 << 8), 1 | (4 << 8) | WROWS))
    for lanes in (1, 2, 8, 16, 32):
        check("reduction %d lanes per row" % lanes,
              gen_r(8, GA_FLOAT, GA_FLOAT, GA_LONG, 64 | (lanes << 16), 4, 2 | (2 << 8) | WROWS))
    for cv, src in ((4, GA_FLOAT), (2, GA_DOUBLE), (8, GA_UBYTE)):
        check("reduction %d outputs per lane" % cv,
              gen_r(8 if src != GA_UBYTE else 0, src, src if src != GA_UBYTE else GA_LONG, GA_LONG,
                    256, 1 | (cv << 16), 4))
    for op, src in ((8, GA_FLOAT), (4, GA_HALF), (6, GA_INT)):
        check("column min / max in rising index order, op %d type %d" % (op, src),
              gen_r(op, src, src, GA_LONG, 256, 1 | (4 << 16), 4 | (1 << 26)))
        n += 1
    for op, src, cv in ((0, GA_FLOAT, 4), (8, GA_FLOAT, 4), (6, GA_INT, 4), (0, GA_INT, 2)):
        check("column reduction on any alignment and extent, op %d type %d, %d outputs per lane" % (op, src, cv),
              gen_r(op, src, GA_LONG if (op == 0 and src == GA_INT) else src, GA_LONG, 256, 1 | (cv << 16),
                    4 | (1 << 31) | ((1 << 26) if op in (6, 8) else 0)))
        n += 1
    for op, src, cv, loose in ((0, GA_FLOAT, 4, 1), (6, GA_INT, 4, 0), (0, GA_DOUBLE, 2, 0), (0, GA_HALF, 1, 0)):
        check("column reduction with neighbouring groups on one die, op %d type %d, %d outputs per lane" % (op, src, cv),
              gen_r(op, src, src, GA_LONG, 256, 1 | (cv << 16) | (1 << 24),
                    4 | ((1 << 31) if loose else 0) | ((1 << 26) if op in (6, 8) else 0)))
        n += 1
    for op, cv in ((13, 16), (12, 4), (13, 8)):
        check("column any / all over bytes, op %d, %d outputs per lane" % (op, cv),
              gen_r(op, GA_UBYTE, GA_BOOL, GA_LONG, 256, 1 | (cv << 16), 4))
        n += 1
    for lo in (4, 16):
        check("reduction %d outer coordinates side by side" % lo,
              gen_r(8, GA_FLOAT, GA_FLOAT, GA_LONG, 64, 4, 4 | (lo << 16)))
    for op, src in ((0, GA_FLOAT), (8, GA_FLOAT), (13, GA_UBYTE), (0, GA_HALF)):
        check("reduction rows read from the boundary below their start, op %d type %d" % (op, src),
              gen_r(op, src, GA_BOOL if op == 13 else GA_FLOAT, GA_LONG, 256, 4 if src == GA_FLOAT else 8,
                    4 | (1 << 24)))
    for op, src, d0 in ((0, GA_FLOAT, GA_FLOAT), (8, GA_FLOAT, GA_FLOAT), (13, GA_UBYTE, GA_BOOL),
                        (0, GA_HALF, GA_FLOAT), (4, GA_DOUBLE, GA_DOUBLE), (0, GA_INT, GA_LONG)):
        check("reduction short rows staged in LDS, op %d type %d" % (op, src),
              gen_r(op, src, d0, GA_LONG, 64, 1, 1 | (1 << 25)))
        n += 1
    # ops: 0 sum, 4 max, 8 maxandargmax, 6 argmax (the enum of reduction.h), 13 any
    for op, src, d0, te in ((0, GA_FLOAT, GA_FLOAT, 3), (8, GA_FLOAT, GA_FLOAT, 5), (13, GA_UBYTE, GA_BOOL, 12),
                            (0, GA_HALF, GA_FLOAT, 6), (4, GA_DOUBLE, GA_DOUBLE, 3), (0, GA_INT, GA_LONG, 2),
                            (0, GA_UBYTE, GA_LONG, 30)):
        check("reduction tiny rows in registers, op %d type %d, %d elements" % (op, src, te),
              gen_r(op, src, d0, GA_LONG, 64, te, 1 | (1 << 29)))
        n += 1
    for op, src, d0 in ((0, GA_FLOAT, GA_FLOAT), (0, GA_HALF, GA_FLOAT), (0, GA_INT, GA_LONG), (4, GA_INT, GA_INT),
                        (1, GA_DOUBLE, GA_DOUBLE), (13, GA_INT, GA_BOOL), (0, GA_HALF, GA_HALF)):
        check("reduction over leading dims with short kept rows in one launch, op %d type %d" % (op, src),
              gen_r(op, src, d0, GA_LONG, 64, 1, 8 | (1 << 30)))
        n += 1
    GA_BYTE, GA_ULONG = 1, 8
    for label, spec in (("sum of unsigned bytes", (0, GA_UBYTE, GA_ULONG, GA_LONG, 256, 16, 8)),
                        ("sum of signed bytes", (0, GA_BYTE, GA_LONG, GA_LONG, 256, 16, 8)),
                        ("sum of bytes, shifted rows", (0, GA_UBYTE, GA_ULONG, GA_LONG, 256, 16, 8 | (1 << 24))),
                        ("all over stepped bytes", (12, GA_UBYTE, GA_BOOL, GA_LONG, 64, 8 | (2 << 8), 4 | WROWS))):
        check("reduction four bytes per operation: " + label, gen_r(*spec))
        n += 1
    check("reduction scalar loads", gen_r(8, GA_DOUBLE, GA_DOUBLE, GA_LONG, 64, 1, 8))
    # an expression over several arrays and a scalar feeding the reduction
    margs = (ElemwiseArg * 3)(ElemwiseArg(b"a", GA_FLOAT, 2), ElemwiseArg(b"b", GA_HALF, 2),
                              ElemwiseArg(b"s", GA_FLOAT, 1 | 2))
    m = 0
    for op, red, neu, acc in [(0, None, None, GA_FLOAT), (8, None, None, GA_FLOAT),
                              (14, b"a + b", b"0", GA_DOUBLE), (13, None, None, GA_FLOAT),
                              (14, b"max(a, b)", b"-INFINITY", GA_HALF)]:
        d0 = GA_BOOL if op == 13 else acc
        for G, V, U, mask in [(256, 4, 4, 0b11), (64, 4, 2, 0b01), (64, 4, 2 | WROWS, 0b01), (256, 1, 4, 0b11)]:
            check("map-reduce op=%d G=%d V=%d mask=%x" % (op, G, V, mask),
                  gen_m(op, red, neu, acc, b"", b"s*a*b", 3, margs, d0, G, V, U, mask))
            m += 1
    gen_t = ext(b"hip_take1_source", C.c_void_p, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint])
    t = 0
    for chunks, a_tc, v_tc, i_tc, tnd in [(1, GA_FLOAT, GA_FLOAT, GA_LONG, 1), (0, GA_FLOAT, GA_FLOAT, GA_INT, 1),
                                          (0, GA_DOUBLE, GA_FLOAT, GA_UBYTE, 3), (0, GA_HALF, GA_HALF, GA_LONG, 2),
                                          (0, GA_BOOL, GA_BOOL, GA_LONG, 1), (2, GA_FLOAT, GA_FLOAT, GA_LONG, 1),
                                          (2, GA_FLOAT, GA_FLOAT, GA_UBYTE, 1)]:
        check("take1 chunks=%d types=%d,%d,%d nd=%d" % (chunks, a_tc, v_tc, i_tc, tnd),
              gen_t(chunks, a_tc, v_tc, i_tc, tnd))
        t += 1
    print("device sources compile for gfx950 (%d reduction variants, %d map-reduce, %d take1, "
          "50 elementwise)" % (n + 20, m, t))


if __name__ == "__main__":
    sys.exit(main())
