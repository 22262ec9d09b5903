"""What a compiled code object says about its kernels' registers.

hiprtc returns an ELF code object whose note section carries the AMDGPU metadata (a MessagePack map, note type
32): per kernel the vector and scalar registers it was allocated, how many vector registers the register
allocator had to spill, and the scratch memory that takes.  This is data the compiler publishes about the code it
just generated for us; nothing is decoded from the instructions.
"""
import struct

_NT_AMDGPU_METADATA = 32
_SHT_NOTE = 7


def _notes(data):
    if data[:4] != b"\x7fELF" or data[4] != 2:
        return
    shoff = struct.unpack_from("<Q", data, 0x28)[0]
    shentsize, shnum = struct.unpack_from("<HH", data, 0x3A)
    for i in range(shnum):
        off = shoff + i * shentsize
        sh_type = struct.unpack_from("<I", data, off + 4)[0]
        sh_offset, sh_size = struct.unpack_from("<QQ", data, off + 0x18)
        if sh_type != _SHT_NOTE:
            continue
        p = sh_offset
        while p + 12 <= sh_offset + sh_size:
            namesz, descsz, ntype = struct.unpack_from("<III", data, p)
            p += 12
            name = data[p:p + namesz]
            p += (namesz + 3) & ~3
            desc = data[p:p + descsz]
            p += (descsz + 3) & ~3
            yield name.rstrip(b"\0"), ntype, desc


def kernel_resources(code):
    """{kernel name: {"vgprs", "agprs", "sgprs", "spilled_vgprs", "scratch_bytes", "lds_bytes", "max_threads"}}
    of a gfx9 code object (bytes); empty when the object carries no metadata note."""
    import msgpack
    out = {}
    for name, ntype, desc in _notes(code):
        if name != b"AMDGPU" or ntype != _NT_AMDGPU_METADATA:
            continue
        md = msgpack.unpackb(desc, raw=False, strict_map_key=False)
        for k in md.get("amdhsa.kernels", []):
            out[k[".name"]] = {
                "vgprs": k.get(".vgpr_count", 0), "agprs": k.get(".agpr_count", 0), "sgprs": k.get(".sgpr_count", 0),
                "spilled_vgprs": k.get(".vgpr_spill_count", 0), "scratch_bytes": k.get(".private_segment_fixed_size", 0),
                "lds_bytes": k.get(".group_segment_fixed_size", 0), "max_threads": k.get(".max_flat_workgroup_size", 0),
            }
    return out


def spilled_vgprs(code):
    """Vector registers spilled over all kernels of the code object."""
    return sum(r["spilled_vgprs"] for r in kernel_resources(code).values())
