"""Launch-geometry and code-shape parameters of the emitters, in one place.

The values are the result of measurements on MI355X (256 CUs, wave64, HBM3E):
elementwise kernels do best with one 16-byte access per operand in flight per
thread (more unrolling lowers the achieved bandwidth), row reductions with
four, non-temporal accesses for operand sets larger than the memory-side
cache, and grids large enough that every CU always has several workgroups
queued.
``set(**kw)`` changes a parameter for experiments; kernels are re-planned
because ``signature()`` is part of every kernel memo key.
"""

_params = {
    # flat elementwise kernel
    'flat_block': 1024,         # threads per workgroup
    'flat_unroll': 1,           # vectors per thread per trip
    'flat_blocks_per_cu': 64,   # grid cap, in workgroups per CU
    # Non-temporal hints of the elementwise kernels: True / False for loads and
    # stores alike, or 'auto' = by footprint against the last-level cache
    # (see stream_policy below)
    'flat_stream': 'auto',
    # tiled 2-d elementwise kernel
    'tiled_stream': 'auto',
    'cache_bytes': 256 << 20,   # capacity of the memory-side cache (Infinity Cache)
    # reductions
    'rows_stream': True,       # non-temporal loads: True / False / 'auto' (by footprint);
                               # measured better or equal from 16 MiB inputs upwards
    'rows_unroll': 4,
    'rows_block_mode_bytes': 32768,   # row length from which a workgroup owns a row
    'rows_batch': 2,            # short rows handled per lane group at a time
    'rows_trips': 4,            # ... with up to this many vector loads per lane and row
    'rows_min_group_bytes': 128,  # ... while the lanes of a row still cover this much per load
    'rows_lane_bytes': 128,     # ... and at most this many bytes in flight per lane
    'rows_group_rows_per_lane': 64,   # grid cap for sub-wave groups: CUs * this workgroups
    'cols_stream': True,
    'cols_unroll': 1,
    'scan_stream': 'auto',      # non-temporal hints of the scan kernels
    'scan_waves_per_cu': 32,    # long rows are cut into chunks until this many waves exist
    # fused row-wise functions: words per lane up to which a wave takes a whole row
    'fused_rows_wave_words': 64,
    'target_blocks_per_cu': 8,  # split the reduce axis until the grid has this many
    'min_blocks_per_cu': 2,     # ... but only if it would otherwise have fewer than this
}
_signature = tuple(sorted(_params.items()))
_version = 0


def get(name):
    return _params[name]


def set(**kw):
    global _signature, _version
    for k, v in kw.items():
        if k not in _params:
            raise KeyError(k)
        _params[k] = tuple(v) if isinstance(v, list) else v
    _signature = tuple(sorted(_params.items()))
    _version += 1


def signature():
    return _signature


def stream_policy(setting, in_bytes, out_bytes):
    """(non-temporal loads?, non-temporal stores?) of a launch that reads
    ``in_bytes`` and writes ``out_bytes``.

    'auto': a launch whose operands together exceed the memory-side cache
    streams (both hints on); one that fits uses neither, so that a following
    kernel finds the operands and the result in the cache.  Measured on MI355X
    (copy-like and two-input kernels, 4 MiB to 1 GiB per array, called
    repeatedly on the same arrays, in producer-consumer chains and in the mixed
    benchmark sequence): mixed settings win single cases by up to 10 % but lose
    others by as much, depending on what the neighbouring kernels leave in the
    cache; this rule is never far from the best."""
    if isinstance(setting, (tuple, list)):
        return bool(setting[0]), bool(setting[1])
    if setting != 'auto':
        return bool(setting), bool(setting)
    big = in_bytes + out_bytes > _params['cache_bytes']
    return big, big


def version():
    """Counter of calls to set(): cheap stand-in for signature() in keys
    that only live inside one process."""
    return _version
