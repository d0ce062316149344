"""Write tests/golden/attn_dispatch_cases.json: which (wave, z, h, q block, kv range, flag) the
reference's wave-based attention dispatch gives for every tile id of a few small schedules.

Run once in the build container, where the reference checkout is mounted:

    python tests/golden/make_attn_dispatch_fixtures.py

The reference has no literal table for this mapping, and the kernel it sits in needs Triton's
TLX dialect, so the mapping is taken from the text the reference GENERATES: its
`AnnotationTransformer` (pure Python) rewrites its annotated attention example, and the lines it
emits between "# auto-generated dispatch" and the first use of the pids — together with the
example's own `get_pid_range` — are executed here as ordinary Python, one tile id at a time, the
way the reference's `tests/computation/transform/test_transform_pass.py:220-239` simulates the
GEMM dispatch.  `tl.load / tl.arange / tl.where / tl.min` act on numpy arrays; `dl.wait` records
the flag index.  Nothing of the reference's text is stored: the fixture holds the wave tables
(inputs) and the per-tile tuples (outputs).
"""

import json
import os
import sys
import textwrap

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = os.environ.get("SYNCOPATE_REFERENCE", "/root/reference")

BLOCK_M = BLOCK_N = 128

# name -> (wave_offsets [z, h, q, kv] in elements, wave_sizes, signal_offsets); cum sizes follow
CASES = {
    # Z=2, H=3, two q blocks, one wave: the in-wave order (q fastest, then h, then z)
    "one_wave_z2_h3_q2": ([[0, 0, 0, 0]], [[2, 3, 256, 256]], [-1]),
    # the same heads split over two waves with different kv ranges and flags
    "two_kv_chunks_z2_h3_q2": ([[0, 0, 0, 256], [0, 0, 0, 0]], [[2, 3, 256, 256], [2, 3, 256, 256]], [-1, 0]),
    # waves that start at non-zero z / h / q offsets and differ in shape
    "ragged_offsets": ([[1, 2, 128, 384], [0, 1, 256, 0], [0, 0, 0, 128]],
                       [[1, 2, 384, 128], [2, 1, 128, 384], [1, 3, 256, 256]], [2, -1, 5]),
    # all-gather attention in double-ring arrival order, scaled down: 8 chunks of one kv block
    "double_ring_w8_small": ([[0, 0, 0, o * 128] for o in (0, 1, 7, 6, 4, 5, 3, 2)],
                             [[1, 2, 256, 128]] * 8, [-1, 0, 4, 1, 5, 2, 6, 3]),
}


class Ptr:
    """A device pointer of the generated code: base array + element offset (scalar or vector)."""

    def __init__(self, data, off=0):
        self.data, self.off = np.asarray(data, dtype=np.int64).reshape(-1), off

    def __add__(self, other):
        return Ptr(self.data, self.off + other)

    def __sub__(self, other):
        return Ptr(self.data, self.off - other)


class TL:
    constexpr = int

    @staticmethod
    def arange(lo, hi):
        return np.arange(lo, hi)

    @staticmethod
    def load(ptr):
        # out-of-range lanes of a masked-by-where load (wave_idx - 1 at wave 0) read element 0
        idx = np.clip(ptr.off, 0, len(ptr.data) - 1)
        return ptr.data[idx]

    @staticmethod
    def where(cond, a, b):
        return np.where(cond, a, b)

    @staticmethod
    def min(x):
        return int(np.min(x))


class DL:
    def __init__(self):
        self.waited = None

    def wait(self, ptr, *args, **kwargs):
        self.waited = int(ptr.off)
        return "token"

    @staticmethod
    def consume_token(desc, token):
        return desc


def generated_dispatch():
    sys.path.insert(0, REFERENCE)
    from syncopate.computation.transform.transformer import AnnotationTransformer

    source = open(os.path.join(REFERENCE, "tests/computation/transform/examples/example_attn.py")).read()
    out = AnnotationTransformer(enable_consumer=True, consumer_descriptors=("desc_k", "desc_v")).transform(source)
    lines = out.splitlines()
    begin = next(i for i, l in enumerate(lines) if "# auto-generated dispatch" in l)
    end = next(i for i in range(begin, len(lines)) if lines[i].strip().startswith("start_m"))
    dispatch = textwrap.dedent("\n".join(lines[begin:end]))
    fbegin = next(i for i, l in enumerate(lines) if l.startswith("def get_pid_range"))
    fend = next(i for i in range(fbegin + 1, len(lines)) if lines[i].strip() == "" or lines[i].startswith("@"))
    helper = "\n".join(lines[fbegin:fend])
    return helper, dispatch


def main():
    helper, dispatch = generated_dispatch()
    dispatch_code = compile(dispatch, "<generated dispatch>", "exec")
    result = {"block_m": BLOCK_M, "block_n": BLOCK_N, "cases": {}}
    for name, (offsets, sizes, signals) in CASES.items():
        cum, running = [], 0
        for s in sizes:
            running += s[0] * s[1] * s[2]
            cum.append(running)
        tiles = []
        for tile_id in range(cum[-1] // BLOCK_M):
            dl = DL()
            env = {"tl": TL, "dl": dl, "NUM_WAVES": len(sizes), "BLOCK_M": BLOCK_M, "BLOCK_N": BLOCK_N,
                   "cum_wave_sizes": Ptr(cum), "wave_offsets": Ptr(offsets), "wave_sizes": Ptr(sizes),
                   "signal_offsets": Ptr(signals), "signal_ptr": Ptr([0] * 16), "tile_id": tile_id,
                   "desc_k": None, "desc_v": None}
            exec(helper, env)
            exec(dispatch_code, env)
            tiles.append([int(env[k]) for k in ("wave_idx", "pid_z", "pid_h", "pid_q", "kv_lo", "kv_hi")] +
                         [-1 if dl.waited is None else dl.waited])
        result["cases"][name] = {"wave_offsets": offsets, "wave_sizes": sizes, "cum_wave_sizes": cum,
                                 "signal_offsets": signals, "tiles": tiles}
    path = os.path.join(HERE, "attn_dispatch_cases.json")
    with open(path, "w") as f:
        json.dump(result, f, indent=None, sort_keys=True)
    print(f"wrote {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
