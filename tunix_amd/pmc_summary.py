"""Per-kernel means of one hardware counter from a rocprofv3 counter-collection CSV.

  python -m tunix_amd.pmc_summary <..._counter_collection.csv> FETCH_SIZE [--scale S] [--match TEXT]

prints, for every kernel symbol, the number of dispatches and the mean / max of
the counter over them (times S, the calibration factor of a copy of known
size).  The template arguments of a kernel name are kept, its argument list is
dropped.
"""
import argparse
import collections
import csv
import json


def summarize(path, counter, scale=1.0, match=None):
  agg = collections.defaultdict(list)
  with open(path) as f:
    for row in csv.DictReader(f):
      if row['Counter_Name'] != counter or (match and match not in row['Kernel_Name']):
        continue
      agg[row['Kernel_Name'].split('(')[0]].append(float(row['Counter_Value']) * scale)
  return {k: {'launches': len(v), 'mean': sum(v) / len(v), 'max': max(v)} for k, v in agg.items()}


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument('csv')
  ap.add_argument('counter')
  ap.add_argument('--scale', type=float, default=1.0)
  ap.add_argument('--json', action='store_true')
  ap.add_argument('--top', type=int, default=16)
  ap.add_argument('--match', default=None, help='only kernels whose name contains this text')
  a = ap.parse_args()
  s = summarize(a.csv, a.counter, a.scale, a.match)
  if a.json:
    print(json.dumps(s))
    return
  rows = sorted(s.items(), key=lambda kv: -kv[1]['mean'] * kv[1]['launches'])[:a.top]
  for k, v in rows:
    print(f"{a.counter} {k[:80]:80s} launches {v['launches']:7d} mean {v['mean']:14.1f} max {v['max']:14.1f}")


if __name__ == '__main__':
  main()
