"""bench.py's command line contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_world_size_from_a_launcher_is_refused_too():
    env = dict(os.environ, WORLD_SIZE="2", RANK="0")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          text=True, timeout=120, env=env)
    assert proc.returncode != 0 and "one GPU" in proc.stderr


def test_bench_probe_library_loads():
    """bench.py's memory yardsticks (cubek_amd/csrc/cq_bench_probes.hip): the library is built, exports its entry
    points, and refuses bad arguments before it touches the GPU."""
    import ctypes

    import bench

    assert os.path.exists(bench.PROBES_PATH), "make -C cubek_amd/csrc builds it"
    L = ctypes.CDLL(bench.PROBES_PATH)
    L.cq_probe_run.restype = ctypes.c_int
    L.cq_probe_run.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64,
                               ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64)]
    assert L.cq_probe_run(0, None, None, None, 100, None, None) == -1      # less than one tile
    assert L.cq_probe_run(7, None, None, None, 1 << 20, None, None) == -1  # no such probe
    L.cq_probe_shape.restype = ctypes.c_int
    L.cq_probe_shape.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64,
                                 ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64)]
    assert L.cq_probe_shape(0, None, None, None, 100, 320, None, None) == -1       # less than one tile
    assert L.cq_probe_shape(0, None, None, None, 1 << 20, 0, None, None) == -1     # nothing on the narrow side
    assert L.cq_probe_shape(1, None, None, None, 1 << 20, 1025, None, None) == -1  # narrow side wider than the wide one
    L.cq_probe_transposed.restype = ctypes.c_int
    L.cq_probe_transposed.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                      ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32]
    assert L.cq_probe_transposed(0, 0, 0, None, None, None, None, 100, 256) == -1   # rows not in whole tiles
    assert L.cq_probe_transposed(1, 1, 1, None, None, None, None, 128, 0) == -1     # no columns
