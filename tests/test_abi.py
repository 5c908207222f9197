"""The drop-in boundary, checked without a GPU: the shared and the static
library export, with C linkage, every entry point that include/anode_routines_gpu.h
declares; the header declares the 46 names of the reference's routines_gpu/lib.h
with the reference's parameter lists; host-side contracts (KernelConfig layout,
the power-of-two assertion, exact division, tiling plans) hold.
"""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

from anode_amd import _lib

# name -> parameter kinds before (cfg, stream), transcribed from routines_gpu/lib.h:32-510
# u = uint32_t, f = float, p = device pointer
REFERENCE_ABI = {
    "anode_gpu_batch_mean_3d1_packed_f32": "uuupp",
    "anode_gpu_batch_mean_bwd_3d1_packed_f32": "uuupp",
    "anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32": "uuupp",
    "anode_gpu_batch_var_3d1_packed_f32": "uuufppp",
    "anode_gpu_batch_var_bwd_3d1_packed_f32": "uuupppp",
    "anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32": "uuupppp",
    "anode_gpu_batch_var_bwd_mean_3d1_packed_f32": "uuupppp",
    "anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32": "uuupppp",
    "anode_gpu_batch_norm_3d1_packed_f32": "uuupppp",
    "anode_gpu_batch_norm_bwd_3d1_packed_f32": "uuuppp",
    "anode_gpu_batch_norm_bwd_3d1_packed_accumulate_f32": "uuuppp",
    "anode_gpu_batch_norm_bwd_mean_3d1_packed_f32": "uuuppp",
    "anode_gpu_batch_norm_bwd_mean_3d1_packed_accumulate_f32": "uuuppp",
    "anode_gpu_batch_norm_bwd_var_3d1_packed_f32": "uuuppppp",
    "anode_gpu_batch_norm_bwd_var_3d1_packed_accumulate_f32": "uuuppppp",
    "anode_gpu_batch_norm_bwd_var_v2_3d1_packed_f32": "uuupppp",
    "anode_gpu_batch_norm_bwd_var_v2_3d1_packed_accumulate_f32": "uuupppp",
    "anode_gpu_upcast_u8_packed_u32": "upp",
    "anode_gpu_discrete_one_hot_3d1_packed_f32": "uuupp",
    "anode_gpu_smooth_negative_f1_loss_3d1_packed_f32": "uuufppp",
    "anode_gpu_smooth_negative_f1_loss_3d1_bwd_packed_f32": "uuufpppp",
    "anode_gpu_M1_copy_map_M2_unit_step_map_R_product_reduce_flat_join_f32": "uppp",
    "anode_gpu_leaky_relu_flat_map_f32": "ufpp",
    "anode_gpu_leaky_relu_flat_map_bwd_f32": "ufppp",
    "anode_gpu_copy_flat_map_f32": "upp",
    "anode_gpu_modulus_flat_map_f32": "upp",
    "anode_gpu_square_flat_map_f32": "upp",
    "anode_gpu_sqrt_flat_map_f32": "upp",
    "anode_gpu_positive_clip_flat_map_f32": "upp",
    "anode_gpu_positive_clip_flat_map_bwd_f32": "uppp",
    "anode_gpu_logistic_flat_map_f32": "upp",
    "anode_gpu_logistic_flat_map_bwd_f32": "uppp",
    "anode_gpu_unit_step_flat_map_f32": "upp",
    "anode_gpu_normal_cdf_flat_map_f32": "upp",
    "anode_gpu_tanh_flat_map_f32": "upp",
    "anode_gpu_rcosh2_flat_map_f32": "upp",
    "anode_gpu_dequantize_u8_packed_f32": "uffpp",
    "anode_gpu_softmax_packed_block_f32": "uupp",
    "anode_gpu_softmax_packed_deterministic_f32": "uupp",
    "anode_gpu_softmax_cat_nll_packed_f32": "uuppp",
    "anode_gpu_softmax_cat_nll_bwd_packed_f32": "uupppp",
    "anode_gpu_softmax_cat_nll_bwd_packed_accumulate_f32": "uupppp",
    "anode_gpu_softmax_nd_packed_f32": "uuupp",
    "anode_gpu_softmax_nd_cat_nll_packed_f32": "uuuppp",
    "anode_gpu_softmax_nd_cat_nll_bwd_packed_f32": "uuupppp",
    "anode_gpu_softmax_nd_cat_nll_bwd_packed_accumulate_f32": "uuupppp",
}

_KIND = {ctypes.c_uint32: "u", ctypes.c_float: "f", ctypes.c_void_p: "p", ctypes.c_int: "i"}


def _nm_defined(path, dynamic):
    out = subprocess.run(["nm", "-D" if dynamic else "-g", "--defined-only", path], check=True,
                         capture_output=True, text=True).stdout
    return {line.split()[-1] for line in out.splitlines() if " T " in line}


def test_reference_abi_has_46_entry_points():
    assert len(REFERENCE_ABI) == 46


def test_header_declares_the_reference_abi_with_its_parameter_lists():
    protos = _lib.parse_header()
    for name, kinds in REFERENCE_ABI.items():
        assert name in protos, f"{name} missing from the header"
        restype, argtypes, names = protos[name]
        assert restype is None, f"{name} must return void"
        got = "".join(_KIND[t] for t in argtypes)
        assert got == kinds + "pp", f"{name}: {got} != {kinds}+cfg+stream"
        assert names[-2:] == ["cfg", "stream"]


def test_shared_library_exports_every_declared_symbol_unmangled():
    assert os.path.exists(_lib.LIBRARY_PATH), "run __graft_entry__.build() first"
    exported = _nm_defined(_lib.LIBRARY_PATH, dynamic=True)
    for name in _lib.parse_header():
        assert name in exported, f"{name} declared but not exported"
    assert not any(s.startswith("_Z") and "anode_gpu" in s for s in exported)


def test_static_archive_defines_every_reference_symbol():
    # the artefact anode's build script links by name: static lib `anode_routines_gpu` (build.rs:23)
    assert os.path.basename(_lib.STATIC_LIBRARY_PATH) == "libanode_routines_gpu.a"
    assert os.path.exists(_lib.STATIC_LIBRARY_PATH)
    defined = _nm_defined(_lib.STATIC_LIBRARY_PATH, dynamic=False)
    for name in REFERENCE_ABI:
        assert name in defined


GPUDEVICEMEM_NAMES = {  # the argument lists of the direct FFI calls at src/ops_gpu.rs:7486-7505, 7595-7614, 9592-9600
    "gpudevicemem_sum_packed_deterministic_f32": "upp",
    "gpudevicemem_sum_packed_accumulate_deterministic_f32": "upp",
    "gpudevicemem_bcast_packed_f32": "upp",
    "gpudevicemem_bcast_packed_accumulate_f32": "upp",
    "gpudevicemem_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32": "uuppp",
}


def test_gpudevicemem_link_names_are_exported_from_an_object_of_their_own():
    protos = _lib.parse_header()
    for name, kinds in GPUDEVICEMEM_NAMES.items():
        restype, argtypes, names = protos[name]
        assert restype is None and "".join(_KIND[t] for t in argtypes) == kinds + "pp" and names[-2:] == ["cfg", "stream"]
    assert set(GPUDEVICEMEM_NAMES) <= _nm_defined(_lib.LIBRARY_PATH, dynamic=True)
    # in the archive they are the only definitions of their member, so a link that already has a gpudevicemem
    # never pulls them in
    out = subprocess.run(["nm", "-g", "--defined-only", _lib.STATIC_LIBRARY_PATH], check=True, capture_output=True,
                         text=True).stdout
    member, by_member = None, {}
    for line in out.splitlines():
        if line.endswith(".o:"):
            member = line[:-1]
        elif " T " in line:
            by_member.setdefault(member, set()).add(line.split()[-1])
    owners = [m for m, syms in by_member.items() if syms & set(GPUDEVICEMEM_NAMES)]
    assert owners == ["gpudevicemem_names.o"], owners
    extern_c = {s for s in by_member["gpudevicemem_names.o"] if not s.startswith("_Z") and not s.startswith("__hip")}
    assert extern_c == set(GPUDEVICEMEM_NAMES), extern_c


def test_library_loads_and_reports_symbol_count():
    lib = _lib.load()
    assert lib.symbol("anode_gpu_reference_symbol_count")() == 46
    assert ctypes.sizeof(_lib.KernelConfig) == 8
    assert _lib.KernelConfig.block_sz.offset == 0 and _lib.KernelConfig.max_block_ct.offset == 4


def test_missing_library_fails_loudly(tmp_path):
    with pytest.raises(FileNotFoundError):
        _lib.Library(str(tmp_path / "libanode_routines_gpu.so"))


_ABORT_SNIPPET = r"""
import ctypes, sys
sys.path.insert(0, {root!r})
from anode_amd import _lib
lib = _lib.load()
cfg = _lib.KernelConfig({block}, 64)
# null device pointers: the contract check comes before anything touches the GPU
lib.symbol({name!r})(*{args!r}, ctypes.byref(cfg), None)
print("returned")
"""


@pytest.mark.parametrize("name", [
    "anode_gpu_batch_mean_3d1_packed_f32",
    "anode_gpu_batch_var_3d1_packed_f32",
    "anode_gpu_batch_norm_bwd_var_3d1_packed_accumulate_f32",
    "anode_gpu_smooth_negative_f1_loss_3d1_packed_f32",
])
def test_reduction_entry_points_abort_on_non_power_of_two_block(name):
    # routines_gpu/batch_norm.cu:68, f1.cu:84: assert(check_power_of_2(block_sz)) on the host
    kinds = REFERENCE_ABI[name]
    args = [{"u": 5, "f": 1e-5, "p": None}[k] for k in kinds]
    code = _ABORT_SNIPPET.format(root=_lib.REPO_ROOT, block=100, name=name, args=args)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == -6, (r.returncode, r.stdout, r.stderr)
    assert "not a power of two" in r.stderr and name in r.stderr
    assert "returned" not in r.stdout


_NO_DEVICE_SNIPPET = r"""
import ctypes, sys
sys.path.insert(0, {root!r})
from anode_amd import _lib
lib = _lib.load()
cfg = _lib.KernelConfig(1024, 1024)
take = lib.symbol("anode_gpu_take_last_error")
# with no device visible every allocation fails: a stand-in for an exhausted GPU that needs none
rc = lib.symbol("anode_gpu_reserve_scratch")(None, 1 << 20)
print("reserve", rc, take(), take())
# [12544, 64, 256] needs partial sums: the reduction must give up, record the error and return
lib.symbol("anode_gpu_batch_mean_3d1_packed_f32")(12544, 64, 256, None, None, ctypes.byref(cfg), None)
print("mean", take(), take())
# the entry point that never allocates refuses an oversized shape before it touches the device
# (tuning knob 9 = 0: without lane tiles this shape is cut into 32 sample tiles per channel group)
lib.cdll.anode_gpu_set_tuning(9, 0)
rc = lib.symbol("anode_gpu_batch_mean_var_3d1_packed_noalloc_f32")(1, 65536, 4096, 1e-5, None, None, None,
                                                                   ctypes.byref(cfg), None)
print("noalloc", rc, take())
print("released", lib.symbol("anode_gpu_release_scratch")(None))
print("alive")
"""


def test_scratch_allocation_failure_is_reported_not_fatal():
    # The ABI returns void: when the partial-sum buffer cannot be allocated the call must skip its launch, keep the
    # process alive and leave the error for anode_gpu_take_last_error().  No GPU is involved: the child sees no device.
    env = dict(os.environ, HIP_VISIBLE_DEVICES="", ROCR_VISIBLE_DEVICES="")
    code = _NO_DEVICE_SNIPPET.format(root=_lib.REPO_ROOT)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    out = dict((line.split()[0], line.split()[1:]) for line in r.stdout.splitlines() if line.strip())
    rc, err, again = (int(v) for v in out["reserve"])
    assert rc != 0 and err == rc and again == 0          # reported once, then cleared
    err, again = (int(v) for v in out["mean"])
    assert err != 0 and again == 0
    assert out["noalloc"] == ["1", "0"]                  # refused by size: not a HIP error
    assert out["released"] == ["0"] and "alive" in out
    # (without a device even the stream's capture state cannot be read: refused at that point, before any allocation)
    assert ("cannot allocate the reduction scratch" in r.stderr or "the reduction scratch is not allocated" in r.stderr)
    assert "nothing was enqueued" in r.stderr
    assert "anode_gpu_batch_mean_3d1_packed_f32" in r.stderr
    assert "more than the 4194304 bytes of the static scratch array" in r.stderr


def test_scratch_size_query_bounds_the_plan():
    lib = _lib.load()
    q = lib.symbol("anode_gpu_reduce_scratch_bytes")
    for S, C, N in [(784, 16, 32), (12544, 64, 256), (49, 2048, 256), (1, 1000, 64), (3, 5, 7)]:
        ppcs = [_plan(S, C, N, a)["ppc"] for a in (True, False)]
        assert q(S, C, N) == max(3 * 8 * C * ppc if ppc > 1 else 0 for ppc in ppcs)  # three fp64 sums per partial
    assert q(0, 5, 3) == 0 and q(7, 5, 1) == 0


def test_host_arg_max_follows_the_reference_rule():
    # src/utils/mod.rs:31-41: start from (-inf, 0); strictly greater wins; NaN never wins
    fn = _lib.load().symbol("anode_host_arg_max_f32")

    def arg_max(values):
        a = np.asarray(values, np.float32)
        return fn(a.ctypes.data, a.size)

    assert arg_max([1, 3, 3, 2]) == 1
    assert arg_max([-np.inf, -np.inf]) == 0
    assert arg_max([np.nan, 1.0, np.nan, 1.0]) == 1
    assert arg_max([np.nan, np.nan]) == 0
    assert arg_max([]) == 0
    assert arg_max([-1, -0.0, 0.0]) == 1
    x = np.random.default_rng(0).standard_normal(1000).astype(np.float32)
    assert arg_max(x) == int(np.argmax(x))


def test_exact_division_helper_matches_integer_division():
    probe = _lib.load().cdll.anode_gpu_fastdiv_probe
    g = np.random.default_rng(0)
    divisors = [1, 2, 3, 4, 5, 7, 19, 49, 64, 255, 256, 784, 1000, 12544, 65535, 65536, 65537, 2097152,
                2 ** 31 - 1, 2 ** 31, 2 ** 31 + 1, 2 ** 32 - 1] + [int(v) for v in g.integers(1, 2 ** 32, 40)]
    for d in divisors:
        edge = [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, 2 ** 32 - 1, 2 ** 32 - d, 2 ** 31, 2 ** 31 - 1]
        ns = [n for n in edge if 0 <= n < 2 ** 32] + [int(v) for v in g.integers(0, 2 ** 32, 200)]
        for n in ns:
            assert probe(n, d) == n // d, (n, d)


def _plan(S, C, N, aligned=True):
    out = (ctypes.c_uint32 * 12)()
    _lib.load().cdll.anode_gpu_plan_reduce(S, C, N, int(aligned), out)
    keys = ["whole", "CB", "SB", "n_ctiles", "n_stiles", "NB", "n_ntiles", "ppc", "vec", "grid", "P", "J"]
    return dict(zip(keys, list(out)))


PLAN_SHAPES = [
    (784, 16, 32), (12544, 64, 256), (49, 2048, 256), (2097152, 32, 2), (1, 1000, 64), (1, 1, 1), (3, 5, 7),
    (4097, 3, 9), (4096, 1, 1), (50, 3, 2), (12321, 8, 4), (7, 300000, 2), (100000, 4, 1), (1024, 3, 4), (1023, 7, 4),
    (1025, 5, 3), (196, 512, 64), (300, 64, 32), (2, 3, 1000), (1, 65536, 4096), (255, 9, 2), (257, 9, 2),
    (465, 4, 1),   # 16-byte accesses, C no larger than the channel unit, C*S beyond one pass of the lanes
]


def _check_plan(p, S, C, N, aligned):
    assert p["grid"] == p["n_ctiles"] * p["n_stiles"] * p["n_ntiles"] >= 1
    assert p["ppc"] == p["n_stiles"] * p["n_ntiles"]
    assert (p["n_ntiles"] - 1) * p["NB"] < N <= p["n_ntiles"] * p["NB"]
    if p["vec"]:
        assert aligned
    if p["whole"] == 2:    # lane tiles: CB*S positions fit the 256 lanes of a workgroup, 16 (or 4) bytes per lane
        lanes = 4 if p["vec"] else 1
        assert S <= 256 * lanes and 1 <= p["CB"] <= 256 and p["CB"] * S <= 256 * lanes
        assert (p["n_ctiles"] - 1) * p["CB"] < C <= p["n_ctiles"] * p["CB"]
        assert p["n_stiles"] == 1
        groups = -(-p["CB"] * S // lanes)
        assert p["J"] == 256 // groups >= 1
        if p["vec"]:
            assert (C * S) % 4 == 0 and (p["CB"] == C or (p["CB"] * S) % 4 == 0)
    elif p["whole"] == 1:  # wide tiles
        assert S <= 4096 and p["P"] in (1024, 2048, 4096) and p["CB"] * S <= p["P"] and 1 <= p["CB"] <= 256
        assert (p["n_ctiles"] - 1) * p["CB"] < C <= p["n_ctiles"] * p["CB"]
        assert p["n_stiles"] == 1
        if p["vec"]:
            assert (C * S) % 4 == 0
            assert p["CB"] == C or (p["CB"] * S) % 4 == 0  # every tile starts on a 16-byte boundary
    else:                  # chunk tiles
        assert S > 4096 and p["n_ctiles"] == C
        assert (p["n_stiles"] - 1) * p["SB"] < S <= p["n_stiles"] * p["SB"]
        if p["vec"]:
            assert S % 4 == 0 and (p["SB"] % 4 == 0 or p["n_stiles"] == 1)


@pytest.mark.parametrize("S,C,N", PLAN_SHAPES)
def test_reduction_tiling_covers_the_array_exactly_once(S, C, N):
    for aligned in (True, False):
        p = _plan(S, C, N, aligned)
        _check_plan(p, S, C, N, aligned)
        if not aligned:
            assert not p["vec"]


def test_reduction_tiling_on_drawn_shapes():
    # every branch of the planner on shapes nobody picked: S, C, N log-uniform, both alignments, one and two inputs
    # (a planner bug shows as a failed invariant here, or as a crash of this process: it is host arithmetic)
    g = np.random.default_rng(2024)

    def draw(lo, hi):
        return max(lo, min(hi, int(round(float(np.exp(g.uniform(np.log(lo), np.log(hi + 1))))))))

    done = 0
    while done < 4000:
        S, C, N = draw(1, 3000000), draw(1, 70000), draw(1, 5000)
        if S * C * N >= 2 ** 32:
            continue
        done += 1
        for flags in (0, 1, 2, 3):
            out = (ctypes.c_uint32 * 12)()
            _lib.load().cdll.anode_gpu_plan_reduce(S, C, N, flags, out)
            keys = ["whole", "CB", "SB", "n_ctiles", "n_stiles", "NB", "n_ntiles", "ppc", "vec", "grid", "P", "J"]
            _check_plan(dict(zip(keys, list(out))), S, C, N, bool(flags & 1))


def test_lane_tiles_take_one_launch_for_few_steps_or_many_channel_groups():
    # one partial per channel (no fold kernel, no scratch) where a channel group's samples are at most 64 steps of a
    # workgroup, or where there are at least 256 channel groups; sample tiles and the fold kernel otherwise
    def steps(p, N):
        return -(-N // p["J"])
    for S, C, N in [(784, 16, 32), (196, 32, 32), (49, 64, 32), (1024, 8, 64), (64, 128, 256), (49, 2048, 256)]:
        p = _plan(S, C, N)
        assert p["whole"] == 2 and (steps(p, N) <= 64 or p["n_ctiles"] >= 256), p
        assert p["ppc"] == 1 and p["NB"] == N, p
    for S, C, N in [(784, 16, 128), (784, 16, 4096), (196, 8, 100000)]:
        p = _plan(S, C, N)
        assert p["whole"] == 2 and steps(p, N) > 64 and p["n_ctiles"] < 256 and p["ppc"] > 1, p
    # wide tiles (1024 < S <= 4096) up to 32 steps of 1024 positions (64 with at least 256 channel groups), chunk
    # tiles (S > 4096) up to 56 steps of 1024 floats
    for S, C, N, one in [(3136, 16, 8, True), (2048, 32, 16, True), (3136, 64, 16, False), (3136, 256, 16, True),
                         (4096, 16, 16, False), (12544, 16, 4, True), (12544, 16, 5, False), (50176, 3, 1, False)]:
        p = _plan(S, C, N)
        assert p["whole"] in (0, 1) and (p["ppc"] == 1) == one, (S, C, N, p)


def test_reduction_tiling_without_lane_tiles():
    # tuning knob 9 = 0 switches lane tiles off: short channels then use the wide tiles (in a child process, so that
    # the knob does not leak into other tests)
    code = r"""
import ctypes, json, sys
sys.path.insert(0, %r)
from anode_amd import _lib
lib = _lib.load()
lib.cdll.anode_gpu_set_tuning(9, 0)
out = {}
for d in %r:
    for al in (1, 0):
        buf = (ctypes.c_uint32 * 12)()
        lib.cdll.anode_gpu_plan_reduce(*d, al, buf)
        out["%%d,%%d,%%d,%%d" %% (*d, al)] = list(buf)
print(json.dumps(out))
""" % (_lib.REPO_ROOT, PLAN_SHAPES)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120, check=True)
    import json
    keys = ["whole", "CB", "SB", "n_ctiles", "n_stiles", "NB", "n_ntiles", "ppc", "vec", "grid", "P", "J"]
    for k, v in json.loads(r.stdout).items():
        S, C, N, al = (int(t) for t in k.split(","))
        p = dict(zip(keys, v))
        assert p["whole"] != 2
        _check_plan(p, S, C, N, bool(al))


_HOST_SWEEP = r"""
import ctypes, sys
sys.path.insert(0, {root!r})
import numpy as np
from anode_amd import _lib
from anode_amd._lib import KernelConfig
lib = _lib.load()
cfg = KernelConfig(1024, 1024)
g = np.random.default_rng(5)
def draw(hi):
    return max(1, min(hi, int(round(float(np.exp(g.uniform(0.0, np.log(hi + 1))))))))
calls = 0
for name, (restype, argtypes, pnames) in sorted(lib.prototypes.items()):
    if pnames[-2:] != ["cfg", "stream"]:
        continue
    fn = lib.symbol(name)
    n_dims = sum(1 for t in argtypes[:-2] if t is ctypes.c_uint32)
    for it in range(40):
        while True:
            dims = [0 if g.random() < 0.03 else draw((3000000, 70000, 5000, 100)[min(k, 3)]) for k in range(n_dims)]
            if np.prod([max(d, 1) for d in dims], dtype=object) < 2 ** 32:
                break
        skew = 0 if g.random() < 0.7 else 4      # 16-byte aligned or element-aligned pointers (never dereferenced)
        args, k = [], 0
        for i, t in enumerate(argtypes[:-2]):
            if t is ctypes.c_uint32:
                args.append(dims[k]); k += 1
            elif t is ctypes.c_void_p:
                args.append(0x7f0000001000 + skew + 0x100000 * i)
            else:
                args.append(float(g.uniform(0.01, 2.0)))
        fn(*args, ctypes.byref(cfg), None)
        lib.symbol("anode_gpu_take_last_error")()
        calls += 1
print("calls", calls)
"""


def test_host_side_of_every_entry_point_survives_drawn_shapes():
    # With no device visible every launch fails and is recorded, so what runs is the host arithmetic of each entry
    # point (tiling plans, grids, exact-division constants) on drawn dims and alignments: it must neither trap nor
    # abort.  (A planner once divided by zero at [465, 4, 1].)
    env = dict(os.environ, HIP_VISIBLE_DEVICES="", ROCR_VISIBLE_DEVICES="")
    r = subprocess.run([sys.executable, "-c", _HOST_SWEEP.format(root=_lib.REPO_ROOT)], capture_output=True, text=True,
                       timeout=600, env=env)
    assert r.returncode == 0, (r.returncode, r.stdout[-500:], r.stderr[-2000:])
    assert int(r.stdout.split()[-1]) >= 40 * 90


def test_tuning_defaults():
    # the defaults the measurements were taken with; a knob left out of the initialiser would silently read 0
    # (read in a child process: other tests of this process may have moved a knob)
    code = r"""
import json, sys
sys.path.insert(0, %r)
from anode_amd import _lib
lib = _lib.load()
print(json.dumps([lib.cdll.anode_gpu_set_tuning(k, -1) for k in range(20)]))
""" % (_lib.REPO_ROOT,)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120, check=True)
    import json
    v = json.loads(r.stdout)
    assert v[0] == 0                      # flat maps: one 16-byte group per thread on a full grid
    assert v[1] == -1 and v[19] == -1     # no such knobs
    assert v[3] == 3 and v[4] == 2        # streaming loads and stores in the maps, streaming loads in the reductions
    assert v[5] == 192 << 20 and v[7] == 16 << 20
    assert v[9] == 1 and v[10] == 256 and v[11] == 2048 and v[12] == 128
    assert v[13] == 2                     # n-d NLL backward deals its pixel groups per XCD
    assert v[14] == 131072                # ... and walks planes of up to 131072 pixels as a flat array
    assert v[15] == 3                     # rows of 16385 to 65536 classes: half in LDS, half in registers
    assert v[16] == 32                    # n-d softmax forward at 17 to 24 classes: five workgroups per CU
    assert v[17] == 1                     # n-d softmax, short planes of many classes: whole samples in registers
    assert v[18] == 1                     # n-d softmax, 33 to 512 classes on longer planes: column tiles in registers


def test_product_package_never_reaches_the_oracle():
    # the oracle is test infrastructure: nothing under anode_amd/ may import, load or link it
    root = os.path.join(_lib.REPO_ROOT, "anode_amd")
    for dirpath, _, files in os.walk(root):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")) or f == "Makefile":
                text = open(os.path.join(dirpath, f), "r", errors="ignore").read()
                assert "oracle" not in text.lower(), f"{os.path.join(dirpath, f)} mentions the oracle"
    needed = subprocess.run(["readelf", "-d", _lib.LIBRARY_PATH], capture_output=True, text=True).stdout
    assert "oracle" not in needed


# ---- which kernel the channel-axis softmax takes for a shape (host logic of the library, no device call) ----

ND_FAMILIES = {0: "rows", 1: "sample_reg", 2: "tile", 3: "col_reg", 4: "col_tile", 5: "pixel_per_thread", 6: "groups16",
               7: "singles"}


def _nd_plan(P, C, separate=True):
    out = (ctypes.c_uint32 * 8)()
    _lib.load().cdll.anode_gpu_softmax_nd_plan_probe(P, C, int(separate), out)
    v = list(out)
    return ND_FAMILIES[v[0]], v[1:]


def test_softmax_nd_plan_invariants():
    # Every tiling the planner hands out must hold the classes, fit the workgroup and cover the plane; a shape's
    # family must not depend on whether the arrays are separate, except for planes that are not whole 16-byte groups
    # (whose 16-byte kernels let the last two groups of a plane overlap and so need separate arrays).
    shapes = [(P, C) for P in (1, 2, 4, 7, 8, 9, 16, 36, 49, 64, 100, 127, 128, 129, 132, 169, 196, 225, 256, 324, 400, 512,
                               576, 784, 900, 1001, 1024, 1025, 1028, 2048, 4100, 4225, 16385, 65535, 65536, 131072, 263169,
                               524288, 1 << 26)
              for C in (1, 2, 3, 19, 21, 32, 33, 40, 64, 65, 100, 128, 129, 150, 200, 256, 257, 300, 400, 512, 513, 944,
                        1000, 1024, 1025, 5000)]
    seen = set()
    for P, C in shapes:
        fam, v = _nd_plan(P, C, True)
        fam_alias, _ = _nd_plan(P, C, False)
        seen.add(fam)
        if P % 4 == 0 or fam in ("rows", "tile", "pixel_per_thread", "singles"):
            assert fam_alias == fam, (P, C, fam, fam_alias)
        else:
            assert fam_alias in ("pixel_per_thread", "singles", "tile"), (P, C, fam, fam_alias)
        if fam == "rows":
            assert P == 1
        elif fam == "sample_reg":
            threads, ns, G, PH = v[:4]
            assert P % 4 == 0 and G == P // 4 and threads in (256, 512, 1024) and ns in (8, 16), (P, C, v)
            assert 1 <= PH <= 32 and G * PH <= threads and PH * ns >= C > 32, (P, C, v)
        elif fam == "col_reg":
            threads, ns, Gt, PH, tiles, xcd = v[:6]
            P4 = -(-P // 4)
            assert threads == 512 and ns in (8, 16, 32) and 33 <= C <= 1024, (P, C, v)
            assert P >= 128 or (P >= 16 and C >= 129 and (P % 4 != 0 or C > 512)), (P, C, v)
            assert 1 <= PH <= 32 and Gt * PH <= 512 and PH * ns >= C, (P, C, v)
            assert Gt <= 64 and (tiles - 1) * Gt < P4 <= tiles * Gt, (P, C, v)
            assert Gt == P4 or Gt % 4 == 0, (P, C, v)
            assert xcd == (0 if P % 32 == 0 else 1), (P, C, v)
        elif fam == "col_tile":
            TP, L, tiles = v[:3]
            assert P % 4 == 0 and TP % 4 == 0 and 16 <= TP <= 256 and L == 256 // TP >= 1, (P, C, v)
            assert (tiles - 1) * TP < P <= tiles * TP and (C * TP + 5 * 256) * 4 <= 65536, (P, C, v)
        elif fam == "groups16":
            assert P % 4 == 0 or (P >= 8 and C <= 32), (P, C)
        elif fam == "pixel_per_thread":
            assert 33 <= C <= 128, (P, C)
    assert seen == set(ND_FAMILIES.values()), seen


def test_softmax_nd_plan_known_shapes():
    # the shapes the measurements in the kernel comments were taken at
    assert _nd_plan(524288, 19)[0] == "groups16"                      # config 3b: two lanes per pixel group
    assert _nd_plan(196, 19)[0] == "tile" and _nd_plan(169, 19)[0] == "tile"
    fam, v = _nd_plan(196, 100)
    assert fam == "sample_reg" and v[:4] == [512, 16, 49, 10]
    fam, v = _nd_plan(36, 256)
    assert fam == "sample_reg" and v[:4] == [256, 16, 9, 28]
    fam, v = _nd_plan(65536, 256)
    assert fam == "col_reg" and v[:6] == [512, 16, 32, 16, 512, 0]
    fam, v = _nd_plan(65536, 64)
    assert fam == "col_reg" and v[:6] == [512, 8, 64, 8, 256, 0]
    fam, v = _nd_plan(1024, 64)                                       # plane and sample powers of two: ragged runs
    assert fam == "col_reg" and v[2:5] == [56, 9, 5]
    fam, v = _nd_plan(900, 200)                                       # planes that are not whole lines: one XCD
    assert fam == "col_reg" and v[1] == 8 and v[5] == 1
    assert _nd_plan(4225, 21)[0] == "groups16" and _nd_plan(4225, 21, separate=False)[0] == "singles"
    assert _nd_plan(4225, 150)[0] == "col_reg" and _nd_plan(4225, 150, separate=False)[0] != "col_reg"
    assert _nd_plan(16, 100)[0] == "col_tile" and _nd_plan(65536, 1025)[0] == "groups16"
    assert _nd_plan(16, 944)[0] == "col_reg" and _nd_plan(16, 1025)[0] == "groups16"
    fam, v = _nd_plan(65536, 1000)                                    # 513 to 1024 classes: 32 slots per thread
    assert fam == "col_reg" and v[1:4] == [32, 16, 32]
    fam, v = _nd_plan(49, 300)                                        # short odd planes with many classes: whole planes
    assert fam == "col_reg" and v[1:6] == [16, 13, 32, 1, 1]
