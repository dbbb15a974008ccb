"""Writes tests/golden/handmade_v3.gguf: a GGUF version 3 file assembled field
by field from the published layout of the format (magic, version, counts,
metadata key/value pairs, tensor infos, padding to the alignment, tensor data;
all little endian), without the writer of this repository.  tests/test_gguf.py
checks that the reader returns exactly the values spelled out here.

Run from the repository root: python tests/golden/make_gguf_fixture.py
"""
import os
import struct

HERE = os.path.dirname(os.path.abspath(__file__))

# metadata value types of the format
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)


def gstr(s):                      # a GGUF string: uint64 length, then the bytes (no terminator)
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def kv(key, vtype, payload):      # key string, uint32 value type, value
    return gstr(key) + struct.pack("<I", vtype) + payload


def build():
    kvs = [
        kv("general.architecture", STRING, gstr("llama")),
        kv("general.alignment", U32, struct.pack("<I", 32)),
        kv("llama.context_length", U32, struct.pack("<I", 4096)),
        kv("llama.block_count", U32, struct.pack("<I", 32)),
        kv("llama.attention.head_count", U32, struct.pack("<I", 32)),
        kv("llama.attention.layer_norm_rms_epsilon", F32, struct.pack("<f", 1e-5)),
        # value types a loader has to step over
        kv("x.u8", U8, struct.pack("<B", 200)),
        kv("x.i16", I16, struct.pack("<h", -2)),
        kv("x.bool", BOOL, struct.pack("<B", 1)),
        kv("x.u64", U64, struct.pack("<Q", 1 << 40)),
        kv("x.f64", F64, struct.pack("<d", 0.5)),
        # an array of three strings, and an array of two int32
        kv("tokenizer.ggml.tokens", ARRAY, struct.pack("<IQ", STRING, 3) + gstr("<unk>") + gstr("<s>") + gstr("ab")),
        kv("x.i32s", ARRAY, struct.pack("<IQ", I32, 2) + struct.pack("<ii", -7, 9)),
    ]
    # tensor infos: name, uint32 n_dims, uint64 dims (innermost first), uint32 ggml type, uint64 offset into the data
    # section.  An F32 vector of 4 weights, a Q8_0 matrix of 2 rows x 32 columns (one 34-byte block per row), and an
    # F16 matrix of 2 rows x 3 columns.
    norm = struct.pack("<4f", 1.0, -2.0, 0.5, 3.25)
    blocks = b""
    for row in range(2):
        scale = struct.pack("<e", 0.25 * (row + 1))                 # fp16 d
        quants = bytes((i * (row + 1) - 16) & 0xff for i in range(32))   # int8 q[32]
        blocks += scale + quants
    halves = struct.pack("<6e", 1.0, -0.5, 65504.0, 6.1035e-05, 0.0, -2.75)   # row 0, then row 1
    infos = (gstr("output_norm.weight") + struct.pack("<I", 1) + struct.pack("<Q", 4) + struct.pack("<IQ", 0, 0)
             + gstr("blk.0.attn_q.weight") + struct.pack("<I", 2) + struct.pack("<QQ", 32, 2)
             + struct.pack("<IQ", 8, 32)                             # second tensor at the next multiple of 32
             + gstr("blk.0.attn_k.weight") + struct.pack("<I", 2) + struct.pack("<QQ", 3, 2)
             + struct.pack("<IQ", 1, 128))                           # 32 + 68 bytes of blocks, padded to 128
    head = b"GGUF" + struct.pack("<I", 3) + struct.pack("<Q", 3) + struct.pack("<Q", len(kvs)) + b"".join(kvs) + infos
    head += b"\0" * ((-len(head)) % 32)
    data = norm + b"\0" * 16 + blocks + b"\0" * 28 + halves
    return head + data, norm, blocks, halves


if __name__ == "__main__":
    raw, _, _, _ = build()
    with open(os.path.join(HERE, "handmade_v3.gguf"), "wb") as f:
        f.write(raw)
    print("handmade_v3.gguf:", len(raw), "bytes")
