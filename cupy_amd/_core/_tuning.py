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
    # Grid cap, in workgroups per CU.  A workgroup per 16 KiB of every operand
    # and no loop is best at every size measured; with the cap at 64 arrays of
    # 1 GiB looped four times and lost six points (copy 76.6 -> 82.2 % of peak,
    # saxpy 73.7 -> 80.4 %; 256 MiB arrays, which fit under either cap: 83 / 82 %)
    'flat_blocks_per_cu': 1024,
    # Threads per workgroup of a launch that only writes (fill 256 MiB: 70.7 %
    # of peak with 1024, 76.7 % with 256; 1 GiB: 76.8 -> 84.5 %)
    'flat_fill_block': 256,
    # matrices stored row after row combined with a value per row or per column
    # stay in the flat kernel (row and column by one division per vector)
    'flat_bcast': True,
    # matrices whose rows are spaced apart (windows, every second row or
    # column) are walked row by row in vectors instead of in square tiles
    'rows2d': True,
    # ndarray.copy() of an array stored in one piece: the driver's device-to-device
    # copy below this many bytes, the flat elementwise kernel from there on
    # (64 MiB: 23.8 -> 19.8 us, 256 MiB: 98.4 -> 85.5 us; under 32 MiB the call is
    # bound by the host either way and the driver's copy costs it 1.5 us less)
    'copy_kernel_min_bytes': 1 << 25,
    # the pieces of a concatenation whose layouts allow it are copied by one
    # launch (up to eight per launch) instead of a launch each
    'concatenate_one_launch': True,
    # ... by workgroups of this many threads, each moving this many vectors
    'concatenate_block': 256,
    'concatenate_unroll': 1,
    # ... with shorter vectors for rows of fewer than 12 vectors, so that no row
    # ends in a partial one (window of 7 columns: 235 -> 142 us; from 12
    # vectors per row on, the partial vector costs less than shorter accesses)
    'rows2d_narrow_vec': True,
    # Operands of different widths: the widest moves 16 bytes per access
    # ('wide'; the narrower ones then move less, but consecutive lanes stay on
    # consecutive addresses in every operand) or the narrowest does ('narrow';
    # a lane of the wide operand then covers 32-128 bytes and each access of a
    # wave is spread over four times its size).  Measured on 2^26 elements,
    # narrow -> wide: float32 > 0 -> bool 54 -> 79 % of peak, int8 -> int64
    # 17 -> 77 %, where(mask, float32, float32) 38 -> 83 %, isnan(float64)
    # 52 -> 82 %, float32 * float16 70 -> 79 %.
    'flat_vec_by': 'wide',
    # ... with this many vectors per thread and trip when one array is read and
    # one written (2: +2 to +20 points over 1 there; with three or more arrays
    # 1 is better by 2 to 6 points)
    'flat_mixed_unroll': 2,
    # Non-temporal hints of the elementwise kernels: True / False for loads and
    # stores alike, or 'auto' = by footprint against the last-level cache
    # (see stream_policy below)
    'flat_stream': 'auto',
    # tiled 2-d elementwise kernel
    'tiled_stream': 'auto',
    'tiled_batch_first': True,  # batched tiles: near batch entries before far rows
    'tiled_narrow_elements': 0,      # ... of about this many elements (0: 1536 to 6144 by the width)
    'tiled_flat_stage': True,   # ... read as one contiguous piece where the lines are no whole vectors
    'tiled_narrow': True,       # tiles as narrow as the array where an axis has at most 32 elements
    'tiled_unaligned': True,    # vectors whatever the alignment of rows and columns
    'tiled_tile': None,         # (rows, columns, threads) of a staged tile; None: by shape
    'tiled_xcd': 'auto',        # tiles numbered die by die: 'auto' (operands off the cache lines), True, False
    'tiled_xcd_strip': 16,      # ... a die walking strips of this many tiles across (transposed copy of 8191 x 8193 float32: 136 us in diagonal order, 116 / 110 / 108 / 105 / 118 with strips of 2 / 4 / 8 / 16 / 64)
    'order_by_outputs': True,   # problems of three and more axes are walked in the order their outputs are stored in
    'packed_tiles': 'auto',     # tiles over several axes for 3-d and 4-d problems: 'auto' where tiles of two axes would be small, True wherever they apply, False never
    'packed_order': 'out',      # ... numbered along the axes of the outputs ('out') or of the staged inputs ('in'), fastest first
    'packed_short_rows_bytes': 64,   # ... also for matrices whose rows are shorter than this and do not merge into one run
    'packed_tile_bytes': 16384,  # ... of about this many bytes per array
    'packed_threads': 256,      # ... a workgroup of this many threads each
    'packed_xcd': 'auto',       # ... numbered die by die: 'auto' where their borders fall inside cache lines
    'packed_tiles_below': 2048,  # ... 'auto': where the two tiled axes together hold fewer elements than this
    'tiled_big_min': 256,       # extent of both tile axes from which tiles are 128 x 128
    'cache_bytes': 256 << 20,   # capacity of the memory-side cache (Infinity Cache)
    # reductions
    'rows_stream': True,       # non-temporal loads: True / False / 'auto' (by footprint);
                               # measured better or equal from 16 MiB inputs upwards
    'rows_unroll': 4,
    'rows_block': 256,          # threads of a workgroup that owns a row
    'rows_split_min_trips': 4,  # a split row leaves every workgroup at least this many trips
    'rows_block_grid_per_cu': 0,   # workgroups per CU when a workgroup owns a row (0: one per row)
    'rows_block_mode_bytes': 32768,   # row length from which a workgroup owns a row
    'rows_batch': 2,            # short rows handled per lane group at a time
    'rows_trips': 2,            # ... with up to this many vector loads per lane and row (sum / argmax over 2^20 rows of 128 int32: 87 / 88 us with 1, 77 / 78 with 2, 81 / 82 with 4; rows of 100 float32: 75 / 84, 66 / 67, 74 / 84)
    'rows_min_group_bytes': 128,  # ... while the lanes of a row still cover this much per load
    'rows_lane_bytes': 128,     # ... and at most this many bytes in flight per lane
    # short rows stored back to back go through the LDS: 'auto' (when a lane
    # group per row would idle or load element by element), True (whenever
    # the rows are short enough), False (never)
    'rows_flat': 'auto',
    'rows_flat_max_bytes': 2048,
    # Grid cap for sub-wave groups: CUs * this workgroups (2^28 elements in rows
    # of 1024: sum 83.2 -> 86.4 % of peak, argmax 82.8 -> 86.4 % with 256 instead of 64)
    'rows_group_rows_per_lane': 256,
    'cols_stream': True,
    # Row-slices a thread of the column kernel loads before it uses the first:
    # 1 when the reduce axis is split across workgroups and the rows start on
    # cache-line boundaries (the slices of one thread are then far apart:
    # 16384 x 4096 float32, axis 0: 45.8 us with 1, 50.2 us with 4), otherwise
    # `cols_unroll_near` (64 x 64 x 16384, axis 1: 56.0 -> 47.8 us; 257 x 511 x
    # 509: 78.5 -> 60.6 us)
    'cols_unroll': 1,
    # Narrow dense matrices (2 to 256 columns, except rows of whole vectors that
    # fill a power-of-two group of lanes) are walked as one contiguous piece
    # of memory when reduced down their columns, the columns a lane meets
    # repeating from trip to trip.  'always': every width, whatever the column
    # kernel would make of it (for tests).
    'reduce_via_copy': True,    # reductions over interleaved kept and reduced axes: copy with the reduced axes last, then reduce rows
    'reduce_via_copy_min': 1 << 18,   # ... from this many elements
    'cols_state_bytes_per_lane': 128,   # column reductions: widest vector whose per-column states fit this many bytes of a lane's registers
    'cols_flat': True,
    'cols_flat_min_bytes': 1 << 20,
    # ... every workgroup a run of consecutive trips (one contiguous piece of
    # memory) rather than every grid-th trip, three workgroups per CU: main
    # kernel over 2^26 float32 with 67 / 129 / 200 / 255 columns 41.7 / 40.7 /
    # 39.5 / 40.5 us against 44.6 / 45.6 / 43.1 / 46.6 side by side with five
    # (two per CU: 39.1 / 47.5 / 52.4 / 40.0 -- uneven)
    'cols_flat_chunked': True,
    'cols_flat_blocks_per_cu': 3,
    'cols_flat_block': 0,       # threads of its workgroups (0: 256; 512 and 1024 measured slower)
    # Lanes across the columns of a workgroup, at most (the rest of its 256
    # threads goes down the reduce axis).  Sums over axis 0 of 16384^2 float32 /
    # 8192^2 float64, timed between other operations on other arrays: 161 / 84 us
    # with 64 lanes, 156 / 81 with 32, 166 / 86 with 16 (same number of workgroups)
    'cols_tx': 32,
    # How far the reduce axis is split, in workgroups per CU.  A CU holds eight
    # workgroups of 256 threads: a grid of more than that many runs its last
    # workgroups alone (16384^2 float32, axis 0, 128 column blocks: 159 us with
    # 16 slices, 208 with 17), and a grid that fills every slot is slower than
    # one that leaves a few free (10 to 12 slices: 151 to 153 us; float64
    # 8192^2: 78.6 to 79.5 against 81.7)
    'cols_target_blocks_per_cu': 5,
    # ... and for a row cut into chunks (sum of all elements).  Every lane has
    # four accesses in flight here, so fewer workgroups saturate the memory:
    # 2^28 float32 in 2048 / 1024 / 512 / 384 / 256 chunks: 161 / 160 / 154 /
    # 155 / 183 us; 2^26 float64: 84 / 83 / 80 / 82 / 93
    'rows_target_blocks_per_cu': 2,
    'cols_unroll_near': 4,
    'cols_xcd': 'auto',         # column blocks numbered die by die: 'auto' (rows off the cache lines), True, False
    'cols_solo_block': 1024,    # workgroup of the thread-per-column variant
    # Grid cap of the scan kernels, in workgroups per CU (cumsum along rows of
    # 1024 float32, 2^28 elements: 74.9 % of peak with 32, 80.2 % with 256)
    'scan_blocks_per_cu': 256,
    'scan_stream': 'auto',      # non-temporal hints of the scan kernels
    'scan_tile': True,          # narrow scanned arrays (2..32 columns) staged through the LDS
    'scan_chunk_reuse': True,   # chunked scans: second reading of the input in reverse order
    'scan_cols_threads_per_cu': 256,   # column scans are cut into chunks below this many threads per CU
    'scan_cols_unaligned': True,   # ... and so do the column scans (the last vector of a row overlaps)
    'scan_rows_unaligned': True,   # row scans use vectors whatever the row length and alignment
    'scan_rows_packed': True,
    'scan_tile_max_inner': 64,  # widest tail the staged kernels take
    'scan_lanes': True,
    'scan_slab': True,          # slices with wide rows that fit the LDS: a workgroup stages whole slices
    'scan_slab_min_inner': None,   # ... for rows wider than this (None: by the shape)
    'scan_slab_long': True,     # ... and longer slices of such rows round by round, a workgroup per slice
    'scan_slab_long_slices_per_cu': 2,   # ... when there are this many slices per CU
    'scan_tile_packed': True,   # slices of few rows and a narrow tail: many to a wave
    'scan_tile_packed_min_slices': 0,   # ... when at least this many slices fit one round of a wave (0: by the shape)
    'scan_complex_as_real': True,   # cumsum of complex arrays: as real arrays with twice the columns
    'scan_cols_vec_bytes': 0,
    'scan_chain_cols': True,    # one-pass kernel for many long columns
    'scan_chain_cols_xcd': 'auto',   # tiles numbered band by band of the columns, a band per compute die: 'auto' (rows off the cache lines), True, False
    'scan_chain_cols_unaligned': True,   # 8-byte vectors whatever the length and alignment of the rows (not in place)
    'scan_chain_cols_short': True,   # ... also for columns of a few hundred rows where a thread per column would take single elements
    'scan_chain_cols_waves': 16,
    'scan_chain_cols_trips': 0,
    'scan_chain_cols_vec_bytes': 0,
    'scan_cols_trips': 0,       # rows a thread of the column kernel requests at a time (0: by shape)
    # Rows from this length on take that kernel however many there are: a
    # workgroup per tile with all of it requested at once, instead of a wave
    # that walks the row round by round (2^26 float32 over rotating buffers:
    # rows of 8192 104 -> 91 us, rows of 4096 98 -> 87; rows of 2048 stay with
    # the wave, 89 us)
    'scan_chain_min_row_bytes': 16384,
    'scan_chain_xcd': 'auto',   # rows of the one-pass row scan dealt out die by die: 'auto' (rows off the cache lines), True, False
    'scan_chain': True,         # a few long rows: one pass, tiles chained through published totals
    # ... with this many waves per tile, each lane keeping fewer vectors for the
    # same tile (2^26 float32 in one row, 128 KiB tiles: 4 waves x 8 parts 102 us,
    # 8 x 4 98, 16 x 2 105; 64 rows of 2^20: 101 / 98 / 109).  A plain copy made
    # the same way -- a workgroup loads a whole tile into registers, then
    # stores it -- reaches 79 % of peak with tiles of 32 KiB, 75 % with 48 KiB
    # and 70 % with 64 to 128 KiB, whatever the order and pacing of the
    # accesses inside the tile, against 81 % for a streaming copy: tiles large
    # enough to make the look-back cheap cost about ten points by themselves
    'scan_chain_waves': 8,
    'scan_chain_min_parts': 1,  # ... each lane keeping at least this many times 4 vectors
    'scan_chain_parts': 0,      # ... a wave holds this many times 4 vectors per lane of its tile
                                # (0: by the size of the input)
    'scan_chain_sleep': 8,      # ... and pauses this many times 64 clocks between two polls
    'scan_chain_spin_limit': 1 << 18,   # polls after which a tile of that kernel gives up waiting
    'scan_waves_per_cu': 32,    # long rows are cut into chunks until this many waves exist
    'scan_chain_max_waste': 1.9,    # rows whose tiles would hold this many times their elements take a wave per row instead (rows of 4099 floats: 127 -> 118 us; at 1.25 rows of 5500 lose: 106 -> 118)
    'scan_whole_max_bytes': 1 << 20,   # column scans of up to 256 rows of arrays up to this size are never cut into chunks
    'scan_whole_slices_waves_per_cu': 4,   # ... slices of fewer than 4096 rows with a narrow tail stay whole from this many on
    # fused row-wise functions: words per lane up to which a wave takes a whole row
    'fused_rows': True,         # row-wise fused functions as one kernel (False: one kernel per piece)
    # (measured with a softmax: rows of 4096 float32 74.7 % of peak with a
    # workgroup per row against 70.9 % with a wave per row; rows of 2048 73 %
    # with a wave against 68 % with a workgroup.  Requesting the next row before
    # the current one is worked on did not help: 62 % against 76 % on rows of 8192)
    'fused_rows_wave_words': 32,
    # Lanes of a short row: as many as it has vectors (1 vector per lane).
    # Fewer lanes with more vectors each would repeat less of the work that is
    # done once per row, but their accesses fall apart: softmax over rows of
    # 100 float32 takes 97 us with 1, 104 with 2, 151 with 4 vectors per lane
    'fused_rows_vectors_per_lane': 1,
    # Short rows in flight per group of lanes (softmax over rows of 100 / 33
    # float32: 98 / 142 us with 1, 94 / 132 with 2, 91 / 127 with 4;
    # x / sqrt(sum(x * x)) over rows of 100 / 33 / 64: 87 / 124 / 78 with 1,
    # 90 / 117 / 76 with 4)
    'fused_rows_in_flight': 4,
    # a float32 division by a value the whole row shares (the sum of a softmax)
    # goes through the value's reciprocal and one correction step
    'fused_rows_reciprocal': True,
    # Grid cap of that kernel, in workgroups per CU (softmax 16384x4096: 94.5 us
    # with 16, 86.0 with 64 or more; rows of 1024: 89.9 -> 85.1; layer
    # normalisation over rows of 100: 110 -> 96)
    'fused_rows_blocks_per_cu': 256,
    # Vector accesses need only the alignment of one element: an access of 16
    # bytes at an address that is a multiple of 4 measures within 4 % of an
    # aligned one (reads of 2^28 bytes: 82 % of peak against 86 %), one at an odd
    # byte address reaches 58 % where element-wide accesses stay below 30 %.
    # False restricts vectors to operands aligned to the whole vector.
    'unaligned_vectors': True,
    'mid_flat_lines_per_lane': 32,
    'reduce_finish': True,      # split reductions of moderate size finish inside the launch that makes the partial results
    'reduce_finish_max_bytes': 16 << 20,   # ... up to this much input (beyond, a second launch is quicker)
    'reduce_finish_round_trips': 4,        # ... and while a finishing lane waits for partial results this often at most
    'reduce_finish_max_slots': 1 << 20,    # ... and up to this many words of partial results
    'reduce_finish_spin_limit': 1 << 22,   # polls before a waiting workgroup gives up
    'mid_flat': True,           # middle-axis reductions of short slices with few columns through the LDS
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


def invalidate_records():
    """Moves the version on without changing a parameter: recorded calls, whose
    keys carry the version, are not replayed again (for memory they name that
    is about to go away)."""
    global _version
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
    cache; this rule is never far from the best.

    A launch that writes far more than it reads (a fill, an outer sum of a
    column and a row) keeps plain stores whatever its size: with nothing
    streaming in, the hint only slows the stores down (column + row into 2^26
    float32: 70 us with it, 41 us without; into 2^28: 252 against 171 us)."""
    if isinstance(setting, (tuple, list)):
        return bool(setting[0]), bool(setting[1])
    if setting != 'auto':
        return bool(setting), bool(setting)
    big = in_bytes + out_bytes > _params['cache_bytes']
    return big, big and 8 * in_bytes >= out_bytes


def version():
    """Counter of calls to set(): cheap stand-in for signature() in keys
    that only live inside one process."""
    return _version
