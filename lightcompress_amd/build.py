"""Build liblcq.so (gfx950 HIP kernels + C ABI) in-tree with hipcc.

    python -m lightcompress_amd.build          # compile every csrc/*.hip, link liblcq.so
    python -m lightcompress_amd.build --incremental   # recompile only what changed

hipcc cross-compiles for gfx950 without a GPU.  The shared object lands next
to this file so it travels with the source tree.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / 'csrc'
OBJ = PKG / 'csrc' / 'build'
LIB = PKG / 'liblcq.so'
HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')

# -ffp-contract=off: the quantizers must round after every arithmetic step.
# packed-fp32 VALU ops are disabled for the device pass (the host pass does
# not know the feature and says so; that warning is harmless).
COMMON = ['--offload-arch=gfx950', '-O3', '-fPIC', '-std=c++17', '-ffp-contract=off',
          '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
          '-Wno-unused-command-line-argument']


def _compile(src: Path, incremental: bool = False) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    out = OBJ / (src.stem + '.o')
    if incremental and out.exists():
        newest = max(p.stat().st_mtime for p in [src, *CSRC.glob('*.h')])
        if out.stat().st_mtime > newest:
            return out
    cmd = [HIPCC, *COMMON, '-c', str(src), '-o', str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = '\n'.join(l for l in r.stderr.splitlines() if 'packed-fp32-ops' not in l)
    if r.returncode != 0:
        raise RuntimeError(f'hipcc failed on {src.name}:\n{err}')
    if err.strip():
        sys.stderr.write(err + '\n')
    return out


def build(jobs: int | None = None, incremental: bool = False) -> Path:
    """Compile every csrc/*.hip and link liblcq.so.  `incremental` (a development convenience) keeps objects that are
    newer than their source and every header."""
    srcs = sorted(CSRC.glob('*.hip'))
    if not srcs:
        raise RuntimeError(f'no HIP sources under {CSRC}')
    jobs = jobs or min(len(srcs), int(os.environ.get('MAX_JOBS', os.cpu_count() or 4)))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda p: _compile(p, incremental), srcs))
    cmd = [HIPCC, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', str(LIB), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f'link failed:\n{r.stderr}')
    return LIB


if __name__ == '__main__':
    print(build(incremental='--incremental' in sys.argv))
