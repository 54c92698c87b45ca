"""Post-processing of the event log a training run leaves (train-profile.csv): the timelines and the throughput
figures the reference's evaluation scripts compute from it.

  collect_train_thpt(log, out)     util/profile/collect_train_thpt.py:1-37: finished micro-batches as
                                   start_timestamp,end_timestamp,batch_size rows
  read_train_profile(log)          util/profile/throughput.py:83-167: per rank, the epoch / global-batch /
                                   micro-batch / restart / wait timelines, parsed from the event names
  eval_throughput(...)             util/profile/throughput.py:10-63: the eight figures over the window in which
                                   inference was active
  eval_throughput_by_epoch(...)    util/profile/throughput.py:66-80

Times are milliseconds, throughputs samples per second.  Plain Python over the csv module: the log of a run is a
few thousand rows.
"""
import csv
import re
from typing import Dict, List, Optional, Sequence, Tuple

_BATCH = re.compile(r'batch_(\d+)_(\d+)_(\d+)')            # epoch, batch, size
_RESTART = re.compile(r'batch_restart_(\d+)_(\d+)')        # epoch, batch
_EPOCH = re.compile(r'epoch_(\d+)_(\d+)')                  # epoch, size
_GLOBAL = re.compile(r'global_batch_(\d+)_(\d+)_(\d+)')    # epoch, batch, size
_WAIT = re.compile(r'wait_valid_batch')


def _rows(path: str) -> List[dict]:
    with open(path, newline='') as f:
        out = []
        for r in csv.DictReader(f):
            if not r.get('name'):
                continue            # the blank line between the ranks' blocks
            r['timestamp'], r['duration'] = float(r['timestamp']), float(r['duration'])
            r['rank'] = int(r['rank']) if r.get('rank') not in (None, '') else 0
            out.append(r)
        return out


def _span(r: dict) -> dict:
    return {'timestamp': r['timestamp'], 'start_time': r['timestamp'], 'duration': r['duration'],
            'end_time': r['timestamp'] + r['duration']}


def read_train_profile(path: str) -> List[Dict[str, List[dict]]]:
    """One dict per rank with the keys 'epoch', 'global_batch', 'batch', 'batch_restart', 'wait_valid_batch'.
    A name is matched at its start, as pandas' str.match does: 'batch_restart_..' and 'batch_exception_..' rows
    are not micro-batches (they do not match batch_<digits>), 'global_batch_..' rows are not either."""
    rows = _rows(path)
    ranks = sorted({r['rank'] for r in rows})
    out = []
    for rank in ranks:
        mine = [r for r in rows if r['rank'] == rank]
        t = {'epoch': [], 'global_batch': [], 'batch': [], 'batch_restart': [], 'wait_valid_batch': []}
        for r in mine:
            name = r['name']
            m = _BATCH.match(name)
            if m:
                t['batch'].append(dict(_span(r), epoch=int(m[1]), batch=int(m[2]), batch_size=int(m[3]), tag=r['tag'],
                                       finished=r['tag'] == 'finish'))
            m = _RESTART.match(name)
            if m:
                t['batch_restart'].append(dict(_span(r), epoch=int(m[1]), batch=int(m[2])))
            if _WAIT.match(name):
                t['wait_valid_batch'].append(_span(r))
            m = _EPOCH.match(name)
            if m:
                t['epoch'].append(dict(_span(r), epoch=int(m[1]), epoch_size=int(m[2])))
            m = _GLOBAL.match(name)
            if m:
                t['global_batch'].append(dict(_span(r), epoch=int(m[1]), batch=int(m[2]), batch_size=int(m[3]),
                                              tag=r['tag'], finished=r['tag'] == 'finish'))
        out.append(t)
    return out


def collect_train_thpt(log: str, output: str) -> int:
    """The finished micro-batches of every rank, in log order; returns how many rows were written."""
    n = 0
    with open(output, 'w') as f:
        f.write('start_timestamp,end_timestamp,batch_size\n')
        for r in _rows(log):
            m = _BATCH.match(r['name'])
            if m and r['tag'] == 'finish':
                f.write('{},{},{}\n'.format(r['timestamp'], r['timestamp'] + r['duration'], int(m[3])))
                n += 1
    return n


def _inside(spans: Sequence[dict], begin: float, end: float) -> List[dict]:
    return [s for s in spans if s['start_time'] >= begin and s['end_time'] <= end]


def eval_throughput(batches: Sequence[dict], infer_begin: float, infer_end: float,
                    restarts: Optional[Sequence[dict]] = None, waits: Optional[Sequence[dict]] = None,
                    verbose: bool = False) -> Tuple[float, float, float, float, int, int, float, float]:
    """(ideal_thpt, real_thpt, avg_batch_time, avg_batch_size, num_finished_batch, num_canceled_batch, waste_pct,
    restart_waste_pct) over the micro-batches that lie inside [infer_begin, infer_end]; eight times -1 for an
    empty timeline.  ideal = samples of finished micro-batches per second of their own run time, real = the same
    samples per second of wall time from the first start to the last end inside the window; waste = run time of
    cancelled micro-batches as a share of that wall time."""
    if not batches:
        return -1, -1, -1, -1, -1, -1, -1, -1
    col = _inside(batches, infer_begin, infer_end)
    done = [b for b in col if b['finished']]
    cancelled = [b for b in col if not b['finished']]
    if not col or not done:
        return -1, -1, -1, -1, -1, -1, -1, -1
    num_image = sum(b['batch_size'] for b in done)
    elapsed = max(b['end_time'] for b in col) - min(b['start_time'] for b in col)
    real_thpt = num_image / elapsed * 1000
    finished_time = sum(b['end_time'] - b['start_time'] for b in done)
    ideal_thpt = num_image / finished_time * 1000
    avg_batch_time = sum(b['duration'] for b in done) / len(done)
    avg_batch_size = num_image / len(done)
    cancelled_time = sum(b['duration'] for b in cancelled)
    waste_pct = cancelled_time / elapsed * 100
    if restarts:
        restart_waste = sum(s['duration'] for s in _inside(restarts, infer_begin, infer_end))
        restart_waste_pct = restart_waste / elapsed * 100
    else:
        restart_waste = restart_waste_pct = -1
    if waits:
        wait_waste = sum(s['duration'] for s in _inside(waits, infer_begin, infer_end))
        wait_waste_pct = wait_waste / elapsed * 100
    else:
        wait_waste = wait_waste_pct = -1
    if verbose:
        busy = sum(b['duration'] for b in done)
        print(f"[eval_throughput] elapsed_time {elapsed:.2f} compute {busy:.2f} ({busy / elapsed * 100:.2f}%) "
              f"cancel waste {cancelled_time:.2f} ({waste_pct:.2f}%) "
              f"restart wast {restart_waste:.2f} ({restart_waste_pct:.2f}%) "
              f"wait valid waste {wait_waste:.2f} ({wait_waste_pct:.2f}%) ")
    return (ideal_thpt, real_thpt, avg_batch_time, avg_batch_size, len(done), len(cancelled), waste_pct,
            restart_waste_pct)


def eval_throughput_by_epoch(epochs: Sequence[dict], infer_begin: float, infer_end: float) -> Tuple[float, float, float]:
    """(mean of the per-epoch throughputs, samples of all epochs over the wall time they span, mean epoch time in
    seconds) over the epochs inside the window; three times -1 without any."""
    col = _inside(epochs, infer_begin, infer_end) if epochs else []
    if not col:
        return -1, -1, -1
    per_epoch = [e['epoch_size'] / e['duration'] * 1000 for e in col]
    total = sum(e['epoch_size'] for e in col)
    e2e = total / (max(e['end_time'] for e in col) - min(e['start_time'] for e in col)) * 1000
    return sum(per_epoch) / len(per_epoch), e2e, sum(e['duration'] for e in col) / len(col) / 1000
