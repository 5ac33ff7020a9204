"""Builds libmbx.so (the HIP kernels + C ABI) and libmbx_probe.so (measurement aids for bench.py) in-tree for
gfx950 with hipcc.

    python megablocks_amd/build.py            # compile what is out of date
    python megablocks_amd/build.py --force    # recompile everything

(run it as a script: `python -m megablocks_amd.build` would import the package, which needs the
library to exist already)
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
BUILD = os.path.join(HERE, 'build')
LIB = os.path.join(HERE, 'libmbx.so')
PROBE_LIB = os.path.join(HERE, 'libmbx_probe.so')
# the library with per-tile time stamps in the grouped-GEMM kernels (csrc/gmm_dma.h, MBX_TICKS), for bench.py --tile-ticks
TICKS_LIB = os.path.join(HERE, 'libmbx_ticks.so')
PROBE_SOURCE = 'probe.hip'
SOURCES = ['routing.hip', 'permute.hip', 'gmm.hip', 'elementwise.hip', 'router.hip']
HEADERS = [os.path.join(CSRC, 'common.h'), os.path.join(CSRC, 'gmm_dma.h'),
           os.path.join(os.path.dirname(HERE), 'include', 'mbx.h'), os.path.join(os.path.dirname(HERE), 'include', 'mbx_probe.h')]
ARCH = 'gfx950'
# -packed-fp32-ops is switched off: hipcc must not form v_pk_*_f32 from scalar float code.
FLAGS = ['-O3', '-fPIC', '-std=c++17', f'--offload-arch={ARCH}', '-Xclang', '-target-feature', '-Xclang',
         '-packed-fp32-ops', '-Wno-unused-command-line-argument']


def _hipcc():
    for cand in (os.environ.get('HIPCC'), '/opt/rocm/bin/hipcc', 'hipcc'):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return 'hipcc'


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = '\n'.join(l for l in proc.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f'command failed: {" ".join(cmd)}\n{out}')
    return out


def build(force: bool = False, verbose: bool = False) -> str:
    os.makedirs(BUILD, exist_ok=True)
    hipcc = _hipcc()
    objs = []
    newest_header = max(os.path.getmtime(h) for h in HEADERS)
    procs = []
    for src in SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(BUILD, src.replace('.hip', '.o'))
        objs.append(o)
        stale = force or not os.path.exists(o) or os.path.getmtime(o) < max(os.path.getmtime(s), newest_header)
        if stale:
            cmd = [hipcc] + FLAGS + ['-c', s, '-o', o]
            if verbose:
                print(' '.join(cmd), flush=True)
            procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    # gmm.hip a second time with the time stamps compiled in
    gmm_src, ticks_obj = os.path.join(CSRC, 'gmm.hip'), os.path.join(BUILD, 'gmm_ticks.o')
    ticks_stale = force or not os.path.exists(ticks_obj) or os.path.getmtime(ticks_obj) < max(os.path.getmtime(gmm_src), newest_header)
    if ticks_stale:
        cmd = [hipcc] + FLAGS + ['-DMBX_TICKS', '-c', gmm_src, '-o', ticks_obj]
        if verbose:
            print(' '.join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    probe_src = os.path.join(CSRC, PROBE_SOURCE)
    probe_cmd = None
    if force or not os.path.exists(PROBE_LIB) or os.path.getmtime(PROBE_LIB) < max(os.path.getmtime(probe_src), newest_header):
        probe_cmd = [hipcc] + FLAGS + ['-shared', probe_src, '-o', PROBE_LIB]
        if verbose:
            print(' '.join(probe_cmd), flush=True)
        procs.append((probe_cmd, subprocess.Popen(probe_cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for cmd, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError(f'command failed: {" ".join(cmd)}\n{out}')
    if [c for c, _ in procs if c is not probe_cmd] or force or not os.path.exists(LIB) or not os.path.exists(TICKS_LIB):
        _run([hipcc, '-shared', '-fPIC', f'--offload-arch={ARCH}', '-o', LIB] + objs)
        _run([hipcc, '-shared', '-fPIC', f'--offload-arch={ARCH}', '-o', TICKS_LIB] +
             [ticks_obj if o.endswith(os.sep + 'gmm.o') else o for o in objs])
    return LIB


if __name__ == '__main__':
    print(build(force='--force' in sys.argv, verbose=True))
