#!/usr/bin/env python3
"""Writes tests/golden/pmx_*.bin: the bytes of two PMX op-parameter blobs as the reference's own serialisers lay them
out, derived by hand (nothing from the reference is imported or run; the FlatBuffers library is not in its tree).

What fixes every byte:
  * the schema: src/ppl/nn/engines/llm_cuda/pmx/schema/llm_cuda_op_params.fbs:14-23 (KeyValueCacheParam), :75-88
    (MultiHeadCacheAttentionParam), :123-145 (union OpParamType, table OpParam, root_type OpParam; no file identifier):
    field i of a table has vtable slot 4 + 2 i, union member k has type tag k (NONE = 0);
  * the call order of the generated code the reference checks in (pmx/generated/llm_cuda_op_params_generated.h:443-463,
    1042-1070, 1545-1553): Create*Param adds the 4-byte fields in REVERSE schema order, then the 1-byte fields in
    reverse order; CreateOpParam adds `value` (offset), then `value_type`; FinishOpParamBuffer calls Finish(root);
  * the published algorithm of flatbuffers::FlatBufferBuilder (C++), restated below: the buffer grows DOWNWARDS;
    a scalar equal to its default is not written; every write is aligned to its size relative to the END of the
    buffer; EndTable writes the soffset, then a vtable just long enough for the highest slot present.
The byte-level expectations are listed in tests/golden/README.md next to each blob."""
import os
import struct

HERE = os.path.dirname(os.path.abspath(__file__))


class Builder:
    """FlatBufferBuilder, the subset these tables use. `buf` holds the bytes written so far in memory order (a write
    PREPENDS); an object's offset is the buffer size right after it was written, i.e. its distance from the end."""

    def __init__(self):
        self.buf = b""
        self.minalign = 1
        self.fields = []  # (vtable slot, offset) of the table being built
        self.max_voffset = 0

    def size(self):
        return len(self.buf)

    def align(self, n):
        self.minalign = max(self.minalign, n)
        self.buf = b"\0" * ((-len(self.buf)) % n) + self.buf

    def push(self, fmt, v):
        self.align(struct.calcsize(fmt))
        self.buf = struct.pack("<" + fmt, v) + self.buf
        return self.size()

    def add_element(self, slot, fmt, v, default=0):
        if v == default:
            return
        off = self.push(fmt, v)
        self.fields.append((slot, off))
        self.max_voffset = max(self.max_voffset, slot)

    def refer_to(self, off):
        self.align(4)
        return self.size() - off + 4

    def add_offset(self, slot, off):
        if off:
            self.add_element(slot, "I", self.refer_to(off))

    def start_table(self):
        return self.size()

    def end_table(self, start):
        vtableoffsetloc = self.push("i", 0)
        self.max_voffset = max(self.max_voffset + 2, 4)
        vt = bytearray(self.max_voffset)
        struct.pack_into("<H", vt, 0, self.max_voffset)
        struct.pack_into("<H", vt, 2, vtableoffsetloc - start)
        for slot, off in self.fields:
            struct.pack_into("<H", vt, slot, vtableoffsetloc - off)
        self.buf = bytes(vt) + self.buf
        self.fields, self.max_voffset = [], 0
        vt_use = self.size()  # (no earlier identical vtable in these buffers: nothing to share)
        pos = len(self.buf) - vtableoffsetloc
        self.buf = self.buf[:pos] + struct.pack("<i", vt_use - vtableoffsetloc) + self.buf[pos + 4:]
        return vtableoffsetloc

    def finish(self, root):
        self.minalign = max(self.minalign, 4)
        self.buf = b"\0" * ((-(len(self.buf) + 4)) % self.minalign) + self.buf
        self.push("I", self.refer_to(root))
        return self.buf


OP_PARAM_TYPE = {"KeyValueCacheParam": 3, "MultiHeadCacheAttentionParam": 10}


def op_param(b, member_type, member):
    start = b.start_table()
    b.add_offset(6, member)  # value
    b.add_element(4, "B", OP_PARAM_TYPE[member_type])  # value_type
    return b.finish(b.end_table(start))


def mhca_blob(num_heads, num_kv_heads, head_dim, is_causal, is_alibi, num_layer, layer_idx, quant_bit, quant_group,
              cache_mode, cache_layout, page_size):
    b = Builder()
    start = b.start_table()
    for slot, v in ((26, page_size), (24, cache_layout), (22, cache_mode), (20, quant_group), (18, quant_bit),
                    (16, layer_idx), (14, num_layer), (8, head_dim), (6, num_kv_heads), (4, num_heads)):
        b.add_element(slot, "i", v)
    b.add_element(12, "B", int(is_alibi))
    b.add_element(10, "B", int(is_causal))
    return op_param(b, "MultiHeadCacheAttentionParam", b.end_table(start))


def kv_cache_blob(num_layer, layer_idx, quant_bit, quant_group, num_repeat, cache_mode, cache_layout, page_size):
    b = Builder()
    start = b.start_table()
    for slot, v in ((18, page_size), (16, cache_layout), (14, cache_mode), (12, num_repeat), (10, quant_group),
                    (8, quant_bit), (6, layer_idx), (4, num_layer)):
        b.add_element(slot, "i", v)
    return op_param(b, "KeyValueCacheParam", b.end_table(start))


CASES = {
    # Llama-3-8B layer 5: every field but is_alibi / cache_mode / cache_layout is non-default
    "pmx_mhca_llama3_8b_layer5.bin": mhca_blob(32, 8, 128, True, False, 32, 5, 8, 8, 0, 0, 128),
    # trailing defaults (cache_mode, cache_layout, page_size all 0): the vtable stops at quant_group
    "pmx_mhca_trailing_defaults.bin": mhca_blob(40, 40, 128, True, False, 40, 0, 8, 8, 0, 0, 0),
    "pmx_kv_cache_layer3_of_32.bin": kv_cache_blob(32, 3, 8, 8, 1, 0, 0, 128),
}

if __name__ == "__main__":
    for name, blob in CASES.items():
        with open(os.path.join(HERE, name), "wb") as f:
            f.write(blob)
        print(name, len(blob), blob.hex())
