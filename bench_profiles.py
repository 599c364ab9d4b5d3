"""Digests rocprofv3 output of ``bench.py`` runs into the summaries under
``profiles/`` and into ``bench_traffic.json``.

``bench.py --plan FILE`` writes which kernels every operation of a step
launches, in order; a step is the same kernel sequence every time, so row k of
a step in the profiler's output belongs to position k of the plan.  Sub-commands
(each prints the table it writes):

  ktrace     per-kernel statistics and per-operation durations from
             ``--kernel-trace --stats`` output
  pmc        HBM bytes per launch from one FETCH_SIZE and one WRITE_SIZE run,
             scaled by the calibration copy; also writes bench_traffic.json
             for the suite 'configs'
  occupancy  waves, wave occupancy per CU and busy fraction from one run with
             SQ_WAVES SQ_WAVE_CYCLES SQ_BUSY_CYCLES GRBM_GUI_ACTIVE
  table      a bench.py JSON line (per_config) as a table, e.g. the streaming
             ceiling or the size curve

The commands that produced the inputs are passed in with ``--command`` and are
printed at the top of every summary.
"""
import argparse
import collections
import csv
import glob
import json
import os
import statistics

ROOT = os.path.dirname(os.path.abspath(__file__))
HBM_PEAK_GBPS = 8000.0
MAX_WAVES_PER_CU = 32          # 4 SIMDs x 8 wave slots on gfx950


def _one(pattern):
    hits = sorted(glob.glob(pattern, recursive=True))
    if not hits:
        raise SystemExit('no file matches %s' % pattern)
    return hits[-1]


def _kernel_rows(path, name_key='Kernel_Name'):
    rows = list(csv.DictReader(open(path)))
    return [r for r in rows if not r[name_key].startswith('__amd')]


def _positions(plan):
    """[(operation name, kernel name, is first kernel of the operation)]"""
    out = []
    for op in plan['operations']:
        for i, k in enumerate(op['kernels']):
            out.append((op['name'], k, i == 0))
    return out


def _split_steps(seq, names, positions, skip):
    """Cuts the dispatch sequence into steps matching the plan's kernel
    sequence; returns per-position lists of rows, ignoring the first ``skip``
    steps found."""
    want = [k for _, k, _ in positions]
    period = len(want)
    per = collections.defaultdict(list)
    i, found = 0, 0
    while i + period <= len(seq):
        if names[i:i + period] == want:
            if found >= skip:
                for k in range(period):
                    per[k].append(seq[i + k])
            found += 1
            i += period
        else:
            i += 1
    if found <= skip:
        raise SystemExit('the plan\'s kernel sequence occurs %d times in the trace '
                         '(need more than %d)' % (found, skip))
    return per, found - skip


def _header(title, commands, extra=''):
    out = ['# ' + title, '']
    if commands:
        out += ['Commands (from the repository root on the MI355X box):', '', '```']
        out += commands
        out += ['```', '']
    if extra:
        out += [extra, '']
    return out


def _write(path, lines):
    text = '\n'.join(lines) + '\n'
    with open(path, 'w') as f:
        f.write(text)
    print(text)


def cmd_ktrace(a):
    plan = json.load(open(a.plan))
    positions = _positions(plan)
    stats = _kernel_rows(_one(os.path.join(a.dir, '**', '*kernel_stats.csv')), 'Name')
    trace = _kernel_rows(_one(os.path.join(a.dir, '**', '*kernel_trace.csv')))
    trace.sort(key=lambda r: int(r['Start_Timestamp']))
    names = [r['Kernel_Name'] for r in trace]
    per, steps = _split_steps(trace, names, positions, a.skip)
    out = _header(a.title, a.command, a.note)
    out += ['`*_kernel_stats.csv` (every launch of the run: warm-up, parity check and timed steps):', '',
            '| Kernel | Calls | Total ms | Average us | % | Min us | Max us |', '|---|---|---|---|---|---|---|']
    for r in stats:
        out.append('| %s | %s | %.3f | %.1f | %s | %.1f | %.1f |' % (
            r['Name'], r['Calls'], int(r['TotalDurationNs']) / 1e6, float(r['AverageNs']) / 1e3,
            r['Percentage'], int(r['MinNs']) / 1e3, int(r['MaxNs']) / 1e3))
    out += ['', 'Per position in the step, from `*_kernel_trace.csv` (the last %d steps; grid in '
            'work-items as rocprofv3 reports it).  Kernels run back to back on one stream: every '
            'kernel starts on whatever its predecessor left in the caches.  "of peak" = the '
            'operation\'s algorithmic bytes / the summed average duration of its kernels / 8 TB/s.' % steps,
            '', '| # | Operation | Kernel | Grid x | Grid y | Workgroup | VGPRs | LDS B | Average us | Min us | Max us | of peak |',
            '|---|---|---|---|---|---|---|---|---|---|---|---|']
    op_bytes = {op['name']: op['bytes'] for op in plan['operations']}
    op_time = collections.defaultdict(float)
    avgs = {}
    for k, (op, kern, first) in enumerate(positions):
        d = [(int(r['End_Timestamp']) - int(r['Start_Timestamp'])) / 1e3 for r in per[k]]
        avgs[k] = sum(d) / len(d)
        op_time[op] += avgs[k]
    total = 0.0
    for k, (op, kern, first) in enumerate(positions):
        r = per[k][0]
        d = [(int(x['End_Timestamp']) - int(x['Start_Timestamp'])) / 1e3 for x in per[k]]
        total += avgs[k]
        frac = '%.1f %%' % (op_bytes[op] / op_time[op] / 1e3 / HBM_PEAK_GBPS * 100) if first else ''
        out.append('| %d | %s | %s | %s | %s | %s | %s | %s | %.1f | %.1f | %.1f | %s |' % (
            k, op if first else '  (continued)', kern, r['Grid_Size_X'], r['Grid_Size_Y'],
            r['Workgroup_Size_X'], r['VGPR_Count'], r['LDS_Block_Size'], avgs[k], min(d), max(d), frac))
    span = []
    last = len(positions) - 1
    for s in range(steps):
        span.append((int(per[last][s]['End_Timestamp']) - int(per[0][s]['Start_Timestamp'])) / 1e3)
    out += ['', 'Sum of the averages: %.1f us per step; first start to last end of a step: %.1f us on '
            'average (the difference is idle time between kernels).' % (total, sum(span) / len(span))]
    _write(a.out, out)


def _counter_by_position(path, counter, positions, skip):
    rows = _kernel_rows(path)
    rows = [r for r in rows if r['Counter_Name'] == counter]
    rows.sort(key=lambda r: int(r['Dispatch_Id']))
    names = [r['Kernel_Name'] for r in rows]
    per, steps = _split_steps(rows, names, positions, skip)
    return {k: [float(r['Counter_Value']) for r in v] for k, v in per.items()}, per


def cmd_pmc(a):
    plan = json.load(open(a.plan))
    positions = _positions(plan)
    fetch, _ = _counter_by_position(_one(os.path.join(a.fetch_dir, '**', '*counter_collection.csv')),
                                    'FETCH_SIZE', positions, a.skip)
    write, _ = _counter_by_position(_one(os.path.join(a.write_dir, '**', '*counter_collection.csv')),
                                    'WRITE_SIZE', positions, a.skip)
    cal = [k for k, (op, kern, _) in enumerate(positions) if op.startswith('calibration copy')]
    if len(cal) != 1:
        raise SystemExit('the plan must contain the calibration copy (bench.py --calibrate)')
    cal = cal[0]
    cal_kib = 262144.0
    cal_f, cal_w = statistics.median(fetch[cal]), statistics.median(write[cal])
    ff, wf = cal_kib / cal_f, cal_kib / cal_w
    out = _header(a.title, a.command,
                  'Calibration: the plain copy kernel `%s` moves %d KiB each way.  FETCH_SIZE reads '
                  '%.1f KiB for it, WRITE_SIZE %.1f KiB, so counter values are scaled by **%.4f** '
                  '(fetch) and **%.4f** (write).' % (positions[cal][1], cal_kib, cal_f, cal_w, ff, wf))
    out += ['| # | Operation | Kernel | FETCH_SIZE KiB (raw, median) | WRITE_SIZE KiB (raw, median) | '
            'HBM read MiB (scaled) | HBM written MiB (scaled) | HBM bytes / algorithmic bytes |',
            '|---|---|---|---|---|---|---|---|']
    op_bytes = {op['name']: op['bytes'] for op in plan['operations']}
    traffic = collections.defaultdict(int)
    rows = []
    for k, (op, kern, first) in enumerate(positions):
        fv, wv = statistics.median(fetch[k]), statistics.median(write[k])
        traffic[op] += round(fv * ff * 1024) + round(wv * wf * 1024)
        rows.append((k, op, kern, first, fv, wv))
    for k, op, kern, first, fv, wv in rows:
        ratio = '%.4f' % (traffic[op] / op_bytes[op]) if first else ''
        out.append('| %d | %s | %s | %.1f | %.1f | %.1f | %.1f | %s |' % (
            k, op if first else '  (continued)', kern, fv, wv, fv * ff / 1024, wv * wf / 1024, ratio))
    if a.note:
        out += ['', a.note]
    _write(a.out, out)
    if a.traffic_json:
        data = {'source': os.path.relpath(a.out, ROOT),
                'scaling': {'FETCH_SIZE': round(ff, 4), 'WRITE_SIZE': round(wf, 4)},
                'hbm_bytes_per_launch': {op: v for op, v in traffic.items()
                                         if not op.startswith('calibration copy')}}
        with open(a.traffic_json, 'w') as f:
            json.dump(data, f, indent=1)
            f.write('\n')


def cmd_occupancy(a):
    plan = json.load(open(a.plan))
    positions = _positions(plan)
    path = _one(os.path.join(a.dir, '**', '*counter_collection.csv'))
    vals = {}
    for c in ('SQ_WAVES', 'SQ_WAVE_CYCLES', 'SQ_BUSY_CYCLES', 'GRBM_GUI_ACTIVE'):
        vals[c], per = _counter_by_position(path, c, positions, a.skip)
    derived = {}
    if a.derived_dir:
        dpath = _one(os.path.join(a.derived_dir, '**', '*counter_collection.csv'))
        for c in ('OccupancyPercent', 'MeanOccupancyPerCU'):
            derived[c], _ = _counter_by_position(dpath, c, positions, a.skip)
    out = _header(a.title, a.command, a.note)
    out += ['Waves = wavefronts launched (SQ_WAVES).  "Waves per CU" = wave slots held, averaged over '
            'the kernel\'s run and over all %d CUs: 4 x SQ_WAVE_CYCLES / (GRBM_GUI_ACTIVE / %d) / CUs '
            '(the CSV holds GRBM_GUI_ACTIVE summed over the %d XCDs); "occupancy" is that as a share '
            'of the %d slots of a CU.  The last two columns are rocprofv3\'s own derived metrics '
            '`MeanOccupancyPerCU` and `OccupancyPercent` from a second run.  Workgroup size, VGPRs '
            'and LDS are what bound the slots a kernel can hold.'
            % (a.cus, a.xcds, a.xcds, MAX_WAVES_PER_CU), '',
            '| # | Operation | Kernel | Workgroup | VGPRs | LDS B | Waves | GPU cycles | '
            'Waves per CU | Occupancy | MeanOccupancyPerCU | OccupancyPercent |',
            '|---|---|---|---|---|---|---|---|---|---|---|---|']
    for k, (op, kern, first) in enumerate(positions):
        r = per[k][0]
        waves = statistics.median(vals['SQ_WAVES'][k])
        wc = statistics.median(vals['SQ_WAVE_CYCLES'][k])
        ga = statistics.median(vals['GRBM_GUI_ACTIVE'][k]) / a.xcds
        mean = 4.0 * wc / ga / a.cus if ga else 0.0
        d1 = '%.1f' % statistics.median(derived['MeanOccupancyPerCU'][k]) if derived else ''
        d2 = '%.0f %%' % statistics.median(derived['OccupancyPercent'][k]) if derived else ''
        out.append('| %d | %s | %s | %s | %s | %s | %d | %d | %.1f | %.0f %% | %s | %s |' % (
            k, op if first else '  (continued)', kern, r.get('Workgroup_Size', ''),
            r.get('VGPR_Count', ''), r.get('LDS_Block_Size', ''),
            waves, ga, mean, 100.0 * mean / MAX_WAVES_PER_CU, d1, d2))
    _write(a.out, out)


def cmd_table(a):
    out = _header(a.title, a.command, a.note)
    for path in a.json:
        line = [l for l in open(path) if l.lstrip().startswith('{')][-1]
        res = json.loads(line)
        ref = {}
        if a.ceiling:
            cl = [l for l in open(a.ceiling) if l.lstrip().startswith('{')][-1]
            for e in json.loads(cl)['per_config']:
                ref[e['name']] = e['gbps']
        entries = res['per_config']
        in_step = bool(entries) and 'inside the step' in entries[0].get('timing', '')
        out += ['`%s`: %s' % (os.path.basename(path), res['config']['workload']), '',
                '| Operation | Algorithmic bytes | %s | min us | GB/s | of 8 TB/s |%s' % (
                    'us inside the step (median of 15 steps)' if in_step
                    else 'us (median of 7 x 10 calls over rotating buffers)',
                    ' us, ten calls in a row on the same arrays |' if in_step else ''),
                '|---|---|---|---|---|---|' + ('---|' if in_step else '')]
        if a.best_variant:
            # 'name [variant]' entries: keep the fastest variant of every name
            best = collections.OrderedDict()
            for e in entries:
                base, _, var = e['name'].partition(' [')
                if base not in best or e['us'] < best[base]['us']:
                    best[base] = dict(e, name=base + (' -- best of the variants: ' + var.rstrip(']')
                                                      if var else ''))
            entries = list(best.values())
        for e in entries:
            out.append('| %s | %d | %.1f | %.1f | %.0f | %.1f %% |%s' % (
                e['name'], e['bytes'], e['us'], e['min_us'], e['gbps'], e['frac'] * 100,
                ' %.1f |' % e['us_repeated_calls'] if in_step else ''))
        out.append('')
        if in_step:
            out += ['Step of %d operations: %.1f us wall time per step (%.0f GB/s over the '
                    'algorithmic bytes), %.1f us as the sum of the kernels\' own durations.' % (
                        len(entries), res['ms_per_step'] * 1e3, res['value'],
                        sum(e['us'] for e in entries)), '']
        if 'launch_us' in res:
            out += ['Host cost per call (us): ' + ', '.join(
                '%s %s' % (k, v['host_enqueue_us']) for k, v in res['launch_us'].items()), '']
    _write(a.out, out)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawTextHelpFormatter)
    sub = ap.add_subparsers(dest='cmd', required=True)

    def common(p):
        p.add_argument('--out', required=True)
        p.add_argument('--title', required=True)
        p.add_argument('--command', action='append', default=[])
        p.add_argument('--note', default='')
        p.add_argument('--skip', type=int, default=1,
                       help='steps at the start of the run to leave out (warm-up)')
    p = sub.add_parser('ktrace')
    common(p)
    p.add_argument('--dir', required=True)
    p.add_argument('--plan', required=True)
    p.set_defaults(fn=cmd_ktrace)
    p = sub.add_parser('pmc')
    common(p)
    p.add_argument('--fetch-dir', required=True)
    p.add_argument('--write-dir', required=True)
    p.add_argument('--plan', required=True)
    p.add_argument('--traffic-json', default='')
    p.set_defaults(fn=cmd_pmc)
    p = sub.add_parser('occupancy')
    common(p)
    p.add_argument('--dir', required=True)
    p.add_argument('--plan', required=True)
    p.add_argument('--cus', type=int, default=256)
    p.add_argument('--xcds', type=int, default=8)
    p.add_argument('--derived-dir', default='')
    p.set_defaults(fn=cmd_occupancy)
    p = sub.add_parser('table')
    common(p)
    p.add_argument('--json', action='append', required=True)
    p.add_argument('--ceiling', default='')
    p.add_argument('--best-variant', action='store_true')
    p.set_defaults(fn=cmd_table)
    a = ap.parse_args()
    a.fn(a)


if __name__ == '__main__':
    main()
