#!/usr/bin/env python3
"""Cut the small golden fixtures out of the reference's committed test data.

Only DATA files are read (binary/text vectors the reference's own tests hold);
nothing from the reference is imported or executed.  Run in the build container:

    python tests/golden/make_fixtures.py [/root/reference]

Writes, next to this script:
  f32_to_f16.txt        the whole 10 575-pair table (safetensors/testdata/f32_to_f16.txt)
  dequant_q4k_in.bin    record 0 (ggml type 12 = Q4_K, 4 blocks, 576 B) of gguf/testdata/dequant_in.bin
  dequant_q4k_ref.bin   its 1024 float32 from ggml's to_float (gguf/testdata/dequant_ref.bin)
  dequant_in.bin        all eleven records of gguf/testdata/dequant_in.bin (Q4_K, Q5_K, Q5_1, Q8_0, IQ4_NL,
                        F32, F16, BF16, Q4_1, Q5_0, Q6_K; 3.7 KB)
  dequant_ref.bin       ggml's to_float of each (18 KB)
  quant_q4k_in.bin      Q4_K round-to-nearest records of llm/testdata/quant_in.bin:
                        all 16 rows of k=2560 and the first 4 rows of k=10240
  quant_q4k_ref.bin     ggml quantize_chunk -> to_float of the same rows (llm/testdata/quant_ref.bin)

Record formats are kept as the reference writes them (reference/dequant_ref.c:21-24,
reference/quant_ref.c:26-31) so the readers in tests/ read either.
"""
import os
import struct
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
here = os.path.dirname(os.path.abspath(__file__))


def out(name, data):
    with open(os.path.join(here, name), "wb") as f:
        f.write(data)
    print(f"{name}: {len(data)} bytes")


# fp16 table: copied whole, it is 148 KB of text pairs.
out("f32_to_f16.txt", open(os.path.join(ref, "safetensors/testdata/f32_to_f16.txt"), "rb").read())


def dequant_record(path, want_type):
    b = open(path, "rb").read()
    o = 0
    while o < len(b):
        typ, n, nbytes = struct.unpack_from("<IIQ", b, o)
        rec = b[o:o + 16 + nbytes]
        o += 16 + nbytes
        if typ == want_type:
            return rec
    raise SystemExit(f"no record of type {want_type} in {path}")


out("dequant_in.bin", open(os.path.join(ref, "gguf/testdata/dequant_in.bin"), "rb").read())
out("dequant_ref.bin", open(os.path.join(ref, "gguf/testdata/dequant_ref.bin"), "rb").read())
out("dequant_q4k_in.bin", dequant_record(os.path.join(ref, "gguf/testdata/dequant_in.bin"), 12))
out("dequant_q4k_ref.bin", dequant_record(os.path.join(ref, "gguf/testdata/dequant_ref.bin"), 12))


def quant_records(path, is_input):
    b = open(path, "rb").read()
    o = 0
    recs = []
    while o < len(b):
        typ, rows, k, im = struct.unpack_from("<IIII", b, o)
        o += 16
        x = b[o:o + rows * k * 4]
        o += rows * k * 4
        if is_input and im:
            o += k * 4
        recs.append((typ, rows, k, im, x))
    return recs


keep_rows = {2560: 16, 10240: 4}
for src, dst, is_in in (("llm/testdata/quant_in.bin", "quant_q4k_in.bin", True),
                        ("llm/testdata/quant_ref.bin", "quant_q4k_ref.bin", False)):
    blob = b""
    for typ, rows, k, im, x in quant_records(os.path.join(ref, src), is_in):
        if typ != 12 or im:
            continue
        r = keep_rows[k]
        blob += struct.pack("<IIII", typ, r, k, 0) + x[:r * k * 4]
    out(dst, blob)
