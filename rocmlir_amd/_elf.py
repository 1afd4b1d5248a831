"""Minimal ELF64 reader: the kernels (global function symbols) of an AMDGPU
code object.  Used by the build to check that every code object holds exactly
the kernel it is named for, and by the tests on what miirBufferGet returns."""
import struct


def kernel_symbols(blob):
    """Names of the global STT_FUNC symbols defined in the ELF image `blob`."""
    if blob[:4] != b"\x7fELF" or blob[4] != 2 or blob[5] != 1:
        raise ValueError("not a little-endian ELF64 image")
    shoff, = struct.unpack_from("<Q", blob, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", blob, 0x3A)
    sections = []
    for i in range(shnum):
        (_name, sh_type, _flags, _addr, offset, size, link, _info, _align,
         entsize) = struct.unpack_from("<IIQQQQIIQQ", blob, shoff + i * shentsize)
        sections.append((sh_type, offset, size, link, entsize))
    names = set()
    for sh_type, offset, size, link, entsize in sections:
        if sh_type not in (2, 11):          # SHT_SYMTAB, SHT_DYNSYM
            continue
        str_off = sections[link][1]
        for j in range(size // entsize):
            st_name, st_info, _other, st_shndx, _value, _size = struct.unpack_from(
                "<IBBHQQ", blob, offset + j * entsize)
            if (st_info & 0xF) == 2 and (st_info >> 4) == 1 and st_shndx != 0:   # FUNC, GLOBAL, defined
                end = blob.index(b"\0", str_off + st_name)
                names.add(blob[str_off + st_name:end].decode())
    return sorted(names)
