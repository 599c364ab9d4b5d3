"""Fused functions that need more than one kernel.

A function with several reductions, or one that combines a reduced value with
an array again, is not a single elementwise or map-reduce kernel.  The
reference hands such functions to its general tracer
(cupy/_core/_fusion_trace.pyx:26-624, _fusion_kernel.pyx:57-381), which emits
one kernel with grid-wide barriers between the passes -- a cooperative launch
that HIP does not offer for run-time compiled code.

Here the recorded graph (``_fusion_graph``) is cut at its reductions: every
reduction, together with all elementwise work that feeds it, becomes one
map-reduce kernel; what remains after the last reduction becomes one
elementwise kernel per result shape, which also writes the argument arrays the
function updated in place.  Intermediate elementwise values are never written
to memory (a value needed by two kernels is computed in both); only reduction
results are, in pool memory, and the kernels run in order on the current
stream.  When all reductions run along the rows of one matrix and a row fits
the registers of a workgroup, ``_fusion_rows`` turns the same pieces into ONE
kernel instead.
"""
from cupy_amd._core import _fusion_emit
from cupy_amd._core.fusion import _collect, _leaf_reader, _reachable


class Piece:
    """One kernel of a plan: ``targets`` computed from ``leaves`` (input arrays,
    scalars and values stored by earlier kernels)."""
    __slots__ = ('kernel', 'leaves', 'targets', 'kwargs', 'reduce', 'stores')

    def __init__(self, name, leaves, targets, reduce=None, stores=()):
        self.leaves = leaves
        self.targets = targets
        self.reduce = reduce
        self.stores = tuple(stores)
        if reduce is not None:
            self.kernel = _fusion_emit.reduction_kernel(name, reduce, leaves, targets)
            self.kwargs = {} if reduce.axis_arg is None else {'axis': reduce.axis_arg}
        else:
            self.kernel = _fusion_emit.elementwise_kernel(name, leaves, targets, stores)
            self.kwargs = {}


class Plan:
    """The kernels of one recorded function, in launch order."""

    def __init__(self, steps, n_values, inputs, returns, single, store_positions):
        self.steps = steps
        self.n_values = n_values
        self.inputs = inputs                # (value order, reader of the call's arguments)
        self.returns = returns              # as fusion._collect takes them
        self.single = single
        self.store_positions = store_positions

    def run(self, *args):
        vals = [None] * self.n_values
        for order, read in self.inputs:
            vals[order] = read(args)
        outs = []
        for step in self.steps:
            if step[0] == 'kernel':
                piece = step[1]
                out = piece.kernel(*[vals[v.order] for v in piece.leaves], **piece.kwargs)
                if len(piece.targets) == 1:
                    vals[piece.targets[0].order] = out
                else:
                    for t, o in zip(piece.targets, out or ()):
                        vals[t.order] = o
            else:
                _, value = step
                base = vals[value.src.order]
                vals[value.order] = base.reshape(value.shape)
        outs = vals
        return _collect(self.returns, outs, args, self.single)


def leaves_of(targets, stored):
    """Values of ``stored`` (orders) that ``targets`` are computed from, in
    creation order."""
    found = {}
    seen = set()
    stack = list(targets)
    while stack:
        v = stack.pop()
        if v.order in seen or v.kind == 'const':
            continue
        seen.add(v.order)
        if v.order in stored:
            found[v.order] = v
            continue
        stack.extend(v.inputs)
    return [found[k] for k in sorted(found)]


def plan(recording, args, name):
    """Cuts a recording into kernels.  Raises NotImplementedError for what has
    no kernel form (the caller then runs the function as written)."""
    roots = recording.roots()
    reach = _reachable(roots)
    stored = set(v.order for v in reach if v.kind in ('array', 'scalar'))
    steps = []
    n_kernels = 0
    for v in reach:
        if v.kind == 'reduce':
            leaves = leaves_of([v.src], stored)
            steps.append(('kernel', Piece('%s_part%d' % (name, n_kernels), leaves, [v],
                                          reduce=v)))
            n_kernels += 1
            stored.add(v.order)
        elif v.kind == 'keepdims':
            steps.append(('view', v))
            stored.add(v.order)
    # what is left: elementwise results and the arrays written in place, one
    # kernel per shape
    returns = []
    pending = {}
    for kind, ref in recording.returns:
        if kind != 'value':
            returns.append((kind, ref))
            continue
        returns.append(('out', ref.order))
        if ref.order not in stored:
            if ref.shape is None:
                raise NotImplementedError('scalar result')
            group = pending.setdefault(ref.shape, ([], []))
            if not any(ref is m for m in group[0]):
                group[0].append(ref)
    for leaf, value in recording.stores:
        pending.setdefault(tuple(leaf.shape), ([], []))[1].append((leaf, value))
    for shape, (targets, stores) in pending.items():
        leaves = leaves_of(targets + [v for _, v in stores], stored)
        for leaf, _ in stores:
            if not any(leaf is m for m in leaves):
                leaves.append(leaf)
        steps.append(('kernel', Piece('%s_part%d' % (name, n_kernels), leaves, targets,
                                      stores=stores)))
        n_kernels += 1
    inputs = [(v.order, _leaf_reader(v)) for v in reach if v.kind in ('array', 'scalar')]
    store_positions = [leaf.source[1] for leaf, _ in recording.stores]
    sequence = Plan(steps, len(recording.values), inputs, returns, recording.single,
                    store_positions)
    if not recording.stores:
        # all reductions along the rows of one matrix, rows short enough for
        # the registers of a workgroup: one kernel that reads the matrix once
        from cupy_amd._core import _fusion_rows
        pieces = [st[1] for st in steps if st[0] == 'kernel']
        row_plan = _fusion_rows.build(reach, pieces, recording.returns, recording.single,
                                      args, name)
        if row_plan is not None:
            # for calls whose arrays are laid out differently from those the
            # kernel was built for
            row_plan.fallback = sequence
            return row_plan
    return sequence
