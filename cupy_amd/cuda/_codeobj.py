"""Reads kernel metadata out of a gfx950 code object (an ELF file).

The AMDGPU metadata note (``NT_AMDGPU_METADATA``, MessagePack) lists every
kernel with the layout of its argument block.  The launch path uses it to
check that a packed argument block has exactly the size the kernel expects
before the block is handed to the GPU, where a mismatch would surface as a
memory fault instead of an exception.
"""
import struct

import msgpack

_NT_AMDGPU_METADATA = 32


def _notes(elf):
    if elf[:4] != b'\x7fELF' or elf[4] != 2:
        raise ValueError('not a 64-bit ELF code object')
    e_shoff, = struct.unpack_from('<Q', elf, 0x28)
    e_shentsize, e_shnum = struct.unpack_from('<HH', elf, 0x3A)
    for i in range(e_shnum):
        off = e_shoff + i * e_shentsize
        sh_type, = struct.unpack_from('<I', elf, off + 4)
        if sh_type != 7:        # SHT_NOTE
            continue
        sh_offset, sh_size = struct.unpack_from('<QQ', elf, off + 0x18)
        pos = sh_offset
        end = sh_offset + sh_size
        while pos + 12 <= end:
            namesz, descsz, ntype = struct.unpack_from('<III', elf, pos)
            pos += 12
            name = elf[pos:pos + namesz].rstrip(b'\0')
            pos += (namesz + 3) & ~3
            desc = elf[pos:pos + descsz]
            pos += (descsz + 3) & ~3
            yield name, ntype, desc


def kernel_metadata(elf):
    """dict: kernel name -> {'kernarg_size', 'explicit_size', 'args', 'vgprs',
    'sgprs', 'lds', 'scratch'}; ``args`` holds (offset, size, value_kind) of the
    explicit arguments."""
    out = {}
    for name, ntype, desc in _notes(elf):
        if name != b'AMDGPU' or ntype != _NT_AMDGPU_METADATA:
            continue
        meta = msgpack.unpackb(desc, raw=False, strict_map_key=False)
        for k in meta.get('amdhsa.kernels', []):
            args = []
            explicit_end = 0
            for a in k.get('.args', []):
                kind = a.get('.value_kind', '')
                if kind.startswith('hidden'):
                    continue
                args.append((a['.offset'], a['.size'], kind))
                explicit_end = max(explicit_end, a['.offset'] + a['.size'])
            out[k['.name']] = {
                'kernarg_size': k.get('.kernarg_segment_size', 0),
                'explicit_size': explicit_end,
                'args': args,
                'vgprs': k.get('.vgpr_count', 0),
                'sgprs': k.get('.sgpr_count', 0),
                'lds': k.get('.group_segment_fixed_size', 0),
                'scratch': k.get('.private_segment_fixed_size', 0),
            }
    return out
