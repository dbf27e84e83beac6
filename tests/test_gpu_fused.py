"""GPU parity of the fused 4-bit AdamW step and the fp32-state step against the CPU oracle,
called through the C ABI (lpmm._native) on torch device memory."""
import numpy as np
import pytest
import torch

from util import assert_codes, assert_params, assert_rel, to_dev, to_np

pytestmark = pytest.mark.gpu

HYPER = dict(beta1=0.9, beta2=0.999, lr=1e-3, wd=0.01, eps=1e-8)


def _native():
    from lpmm import _native

    return _native


def _run_fused_steps(oracle, qmaps, n, steps, seed, grad_fn=None, p_scale=0.02, offset=0, exact_p=False):
    """Runs `steps` fused steps on GPU and oracle from zero state; compares after every step."""
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    rng = np.random.default_rng(seed)
    p_ref = (rng.standard_normal(n) * p_scale).astype(np.float32)
    nb, ng = (n + 1) // 2, (n + 127) // 128
    mc_ref, vc_ref = np.zeros(nb, np.uint8), np.zeros(nb, np.uint8)
    ms_ref, vs_ref = np.zeros(ng, np.float32), np.zeros(ng, np.float32)

    def dev(a):
        # optional element offset makes the device pointers misaligned for the vector path
        buf = torch.empty(a.size + offset, dtype=torch.from_numpy(a).dtype, device="cuda")
        view = buf[offset:]
        view.copy_(torch.from_numpy(a))
        return view

    p, mc, vc, ms, vs = dev(p_ref), dev(mc_ref), dev(vc_ref), dev(ms_ref), dev(vs_ref)
    dqm, dqv = to_dev(qm), to_dev(qv)
    flips = 0
    for s in range(1, steps + 1):
        g_np = grad_fn(rng, n, s) if grad_fn else (rng.standard_normal(n) * 1e-3).astype(np.float32)
        g = dev(g_np)
        st = lib.lpmm_adamw4bit_step(p.data_ptr(), g.data_ptr(), mc.data_ptr(), vc.data_ptr(), ms.data_ptr(),
                                     vs.data_ptr(), dqm.data_ptr(), dqv.data_ptr(), n, HYPER["beta1"],
                                     HYPER["beta2"], HYPER["lr"], HYPER["wd"], HYPER["eps"], float(s),
                                     torch.cuda.current_stream().cuda_stream)
        assert st == 0, lib.lpmm_status_string(st)
        p_before = p_ref.copy()
        oracle.adamw4bit_step(p_ref, g_np, mc_ref, vc_ref, ms_ref, vs_ref, qm, qv, HYPER["beta1"], HYPER["beta2"],
                              HYPER["lr"], HYPER["wd"], HYPER["eps"], float(s))
        torch.cuda.synchronize()
        flips += assert_codes(to_np(mc), mc_ref, n, f"m codes step {s}")
        flips += assert_codes(to_np(vc), vc_ref, n, f"v codes step {s}")
        assert_rel(to_np(ms), ms_ref, f"m scale step {s}")
        assert_rel(to_np(vs), vs_ref, f"v scale step {s}")
        assert_params(to_np(p), p_ref, p_before, f"p step {s}")
        # every step starts from identical inputs: the oracle's parameters go back to the GPU
        p.copy_(torch.from_numpy(p_ref))
        if flips:
            # after a tie flip the two runs legitimately diverge: resynchronise the GPU state
            mc.copy_(torch.from_numpy(mc_ref)); vc.copy_(torch.from_numpy(vc_ref))
            ms.copy_(torch.from_numpy(ms_ref)); vs.copy_(torch.from_numpy(vs_ref))
            p.copy_(torch.from_numpy(p_ref))
    return flips


@pytest.mark.parametrize("n", [4098, 128 * 37, 128 * 1000 + 64, 2048 * 33, 1600 * 4800 // 8, 4096 * 1024 + 2])
def test_fused_step_matches_oracle(oracle, qmaps, n):
    flips = _run_fused_steps(oracle, qmaps, n, steps=5, seed=n)
    print(f"n={n}: tie flips {flips}")


def test_fused_step_odd_and_tiny(oracle, qmaps):
    # the C ABI itself accepts any n >= 1, including odd n (last byte holds one code)
    for n in (1, 2, 7, 127, 129, 4097, 2049 * 3):
        _run_fused_steps(oracle, qmaps, n, steps=3, seed=100 + n)


def test_fused_step_unaligned_pointers(oracle, qmaps):
    for off in (1, 3):
        _run_fused_steps(oracle, qmaps, 128 * 50 + 10, steps=3, seed=7, offset=off)


def test_fused_step_zero_and_outlier_groups(oracle, qmaps):
    """All-zero gradient groups (0/0 -> code 15, scale 0) and groups with a huge outlier."""

    def grad_fn(rng, n, s):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        g[: 128 * 3] = 0.0          # three groups that stay exactly zero
        g[128 * 5 + 17] = 50.0      # one outlier
        g[128 * 6: 128 * 7] = 1e-30  # g*g underflows to a denormal / zero
        if s == 2:
            g[128 * 8: 128 * 9] = 0.0
        return g

    _run_fused_steps(oracle, qmaps, 128 * 64, steps=4, seed=11, grad_fn=grad_fn)


def test_fused_step_heavy_tailed(oracle, qmaps):
    def grad_fn(rng, n, s):
        z = rng.standard_normal((4, n))
        return (z[0] / np.sqrt((z[1] ** 2 + z[2] ** 2 + z[3] ** 2) / 3.0) * 1e-3).astype(np.float32)

    _run_fused_steps(oracle, qmaps, 128 * 4096, steps=6, seed=5, grad_fn=grad_fn)


def test_fp32_step_matches_oracle(oracle):
    nat = _native()
    lib = nat.lib()
    rng = np.random.default_rng(3)
    for n in (1, 1600, 4096, 5000):
        p_ref = (rng.standard_normal(n) * 0.02).astype(np.float32)
        m_ref, v_ref = np.zeros(n, np.float32), np.zeros(n, np.float32)
        p, m, v = to_dev(p_ref), to_dev(m_ref), to_dev(v_ref)
        for s in range(1, 6):
            g_np = (rng.standard_normal(n) * 1e-3).astype(np.float32)
            g = to_dev(g_np)
            st = lib.lpmm_adamw_fp32_step(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), n, 0.9, 0.999,
                                          1e-3, 0.01, 1e-8, float(s), torch.cuda.current_stream().cuda_stream)
            assert st == 0
            oracle.adamw_fp32_step(p_ref, g_np, m_ref, v_ref, 0.9, 0.999, 1e-3, 0.01, 1e-8, float(s))
            torch.cuda.synchronize()
            np.testing.assert_array_equal(to_np(p), p_ref)
            np.testing.assert_array_equal(to_np(m), m_ref)
            np.testing.assert_array_equal(to_np(v), v_ref)


def test_fp16_step_matches_oracle(oracle):
    """lpmm_adamw_fp16_step_multi (p, g, m, v stored as half, arithmetic in float, the update
    reading the moments after their rounding to half) against the float16 restatement of
    adamw_cuda_kernel<at::Half>: several tensors per call, each with its own step, five steps."""
    nat = _native()
    lib = nat.lib()
    rng = np.random.default_rng(31)
    sizes = [1, 7, 1600, 4096, 1025] + [int(k) for k in rng.integers(1, 4097, 70)]
    host, dev = [], []
    for n in sizes:
        arrs = [(rng.standard_normal(n) * 0.02).astype(np.float16), None,
                np.zeros(n, np.float16), np.zeros(n, np.float16)]
        host.append(arrs)
        dev.append([to_dev(a) if a is not None else None for a in arrs])
    for s in range(1, 6):
        steps = [float(s + i % 3) for i in range(len(sizes))]
        for h, d, n in zip(host, dev, sizes):
            h[1] = (rng.standard_normal(n) * 1e-2).astype(np.float16)
            d[1] = to_dev(h[1])
        table = np.array([(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), n, st, 0.0)
                          for d, n, st in zip(dev, sizes, steps)], dtype=nat.ADAMW_FP32_TENSOR)
        st = lib.lpmm_adamw_fp16_step_multi(table.ctypes.data, len(sizes), 0.9, 0.999, 1e-3, 0.01, 1e-8,
                                            torch.cuda.current_stream().cuda_stream)
        assert st == 0
        torch.cuda.synchronize()
        for (p, g, m, v), d, step in zip(host, dev, steps):
            oracle.adamw_fp16_step(p, g, m, v, 0.9, 0.999, 1e-3, 0.01, 1e-8, step)
            np.testing.assert_array_equal(to_np(d[2]), m)
            np.testing.assert_array_equal(to_np(d[3]), v)
            np.testing.assert_array_equal(to_np(d[0]), p)


def test_multi_tensor_matches_single(oracle, qmaps):
    """lpmm_adamw4bit_step_multi over many tensors (more than one launch record) gives the
    same bytes as the oracle run tensor by tensor, each tensor with its own step."""
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(21)
    sizes = [4098 + 2 * i for i in range(60)] + [128 * 700, 2048 * 9 + 130]
    host, devs, recs = [], [], []
    for i, n in enumerate(sizes):
        nb, ng = (n + 1) // 2, (n + 127) // 128
        h = dict(p=(rng.standard_normal(n) * 0.02).astype(np.float32),
                 g=(rng.standard_normal(n) * 1e-3).astype(np.float32),
                 mc=rng.integers(0, 256, nb, dtype=np.uint8), vc=rng.integers(0, 256, nb, dtype=np.uint8),
                 ms=np.abs(rng.standard_normal(ng) * 1e-3).astype(np.float32),
                 vs=np.abs(rng.standard_normal(ng) * 1e-6).astype(np.float32), step=float(1 + i % 7))
        if n % 2:
            h["mc"][-1] &= 0xF
            h["vc"][-1] &= 0xF
        d = {k: to_dev(v) for k, v in h.items() if k != "step"}
        host.append(h); devs.append(d)
        recs.append((d["p"].data_ptr(), d["g"].data_ptr(), d["mc"].data_ptr(), d["vc"].data_ptr(),
                     d["ms"].data_ptr(), d["vs"].data_ptr(), n, h["step"], 0.0))
    table = np.array(recs, dtype=nat.ADAMW4BIT_TENSOR)
    st = lib.lpmm_adamw4bit_step_multi(table.ctypes.data, len(recs), dqm.data_ptr(), dqv.data_ptr(), 0.9, 0.999,
                                       1e-3, 0.01, 1e-8, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    for h, d, n in zip(host, devs, sizes):
        p_before = h["p"].copy()
        oracle.adamw4bit_step(h["p"], h["g"], h["mc"], h["vc"], h["ms"], h["vs"], qm, qv, 0.9, 0.999, 1e-3, 0.01,
                              1e-8, h["step"])
        assert_codes(to_np(d["mc"]), h["mc"], n, "m codes")
        assert_codes(to_np(d["vc"]), h["vc"], n, "v codes")
        assert_rel(to_np(d["ms"]), h["ms"], "m scale")
        assert_rel(to_np(d["vs"]), h["vs"], "v scale")
        assert_params(to_np(d["p"]), h["p"], p_before, "p")


def test_multi_tensor_whole_tiles(oracle, qmaps):
    """110 tensors, every one a whole number of 2048-element tiles (the straight-line variant of
    the kernel), three launch records with tensors of 1 to 5 tiles: every tile finds its tensor
    through the two-level lookup, also across the boundaries of its coarse table."""
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(77)
    sizes = [2048 * int(k) for k in rng.integers(1, 6, 110)]
    host, devs, recs = [], [], []
    for i, n in enumerate(sizes):
        h = dict(p=(rng.standard_normal(n) * 0.02).astype(np.float32),
                 g=(rng.standard_normal(n) * 1e-3).astype(np.float32),
                 mc=rng.integers(0, 256, n // 2, dtype=np.uint8), vc=rng.integers(0, 256, n // 2, dtype=np.uint8),
                 ms=np.abs(rng.standard_normal(n // 128) * 1e-3).astype(np.float32),
                 vs=np.abs(rng.standard_normal(n // 128) * 1e-6).astype(np.float32), step=float(1 + i % 5))
        d = {k: to_dev(v) for k, v in h.items() if k != "step"}
        host.append(h); devs.append(d)
        recs.append((d["p"].data_ptr(), d["g"].data_ptr(), d["mc"].data_ptr(), d["vc"].data_ptr(),
                     d["ms"].data_ptr(), d["vs"].data_ptr(), n, h["step"], 0.0))
    table = np.array(recs, dtype=nat.ADAMW4BIT_TENSOR)
    st = lib.lpmm_adamw4bit_step_multi(table.ctypes.data, len(recs), dqm.data_ptr(), dqv.data_ptr(), 0.9, 0.999,
                                       1e-3, 0.01, 1e-8, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    for i, (h, d, n) in enumerate(zip(host, devs, sizes)):
        p_before = h["p"].copy()
        oracle.adamw4bit_step(h["p"], h["g"], h["mc"], h["vc"], h["ms"], h["vs"], qm, qv, 0.9, 0.999, 1e-3, 0.01,
                              1e-8, h["step"])
        assert_codes(to_np(d["mc"]), h["mc"], n, f"m codes of tensor {i}")
        assert_codes(to_np(d["vc"]), h["vc"], n, f"v codes of tensor {i}")
        assert_rel(to_np(d["ms"]), h["ms"], f"m scale of tensor {i}")
        assert_rel(to_np(d["vs"]), h["vs"], f"v scale of tensor {i}")
        assert_params(to_np(d["p"]), h["p"], p_before, f"p of tensor {i}")


def test_tile_order_with_offset_bases(oracle, qmaps):
    """The kernel hands the tiles of a tensor to the workgroups in runs of 16 inside 1 MB-aligned blocks
    of the parameter's address range.  Tensors of 300-700 tiles whose parameters start 0, 5, 77 and 130
    tiles (and 1028 elements) past a 1 MB boundary, whole-tile and ragged, in one launch: every tile is
    processed exactly once, whatever block it falls into."""
    nat = _native()
    lib = nat.lib()
    qm, qv = qmaps
    dqm, dqv = to_dev(qm), to_dev(qv)
    rng = np.random.default_rng(123)
    arena = torch.empty((1 << 20) // 4 + 2048 * 3200, dtype=torch.float32, device="cuda")
    skip = (-arena.data_ptr() % (1 << 20)) // 4  # elements to the next 1 MB boundary
    offsets = [0, 2048 * 5, 2048 * 77, 2048 * 130, 2048 * 7 + 1028]
    sizes = [2048 * 400, 2048 * 300 + 700, 2048 * 512, 2048 * 700, 2048 * 333 + 64]
    host, devs, recs, cursor = [], [], [], skip
    for off, n in zip(offsets, sizes):
        start = cursor + off
        cursor = (start + n + (1 << 18) - 1) // (1 << 18) * (1 << 18) + skip % (1 << 18)  # next 1 MB boundary
        h = dict(p=(rng.standard_normal(n) * 0.02).astype(np.float32), g=(rng.standard_normal(n) * 1e-3).astype(np.float32),
                 mc=rng.integers(0, 256, (n + 1) // 2, dtype=np.uint8), vc=rng.integers(0, 256, (n + 1) // 2, dtype=np.uint8),
                 ms=np.abs(rng.standard_normal((n + 127) // 128) * 1e-3).astype(np.float32),
                 vs=np.abs(rng.standard_normal((n + 127) // 128) * 1e-6).astype(np.float32))
        d = {k: to_dev(v) for k, v in h.items() if k != "p"}
        d["p"] = arena[start:start + n]
        d["p"].copy_(torch.from_numpy(h["p"]))
        assert (d["p"].data_ptr() % (1 << 20)) // 8192 == (off // 2048) % 128
        host.append(h); devs.append(d)
        recs.append((d["p"].data_ptr(), d["g"].data_ptr(), d["mc"].data_ptr(), d["vc"].data_ptr(),
                     d["ms"].data_ptr(), d["vs"].data_ptr(), n, 3.0, 0.0))
    table = np.array(recs, dtype=nat.ADAMW4BIT_TENSOR)
    st = lib.lpmm_adamw4bit_step_multi(table.ctypes.data, len(recs), dqm.data_ptr(), dqv.data_ptr(), 0.9, 0.999,
                                       1e-3, 0.01, 1e-8, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    for i, (h, d, n) in enumerate(zip(host, devs, sizes)):
        p_before = h["p"].copy()
        oracle.adamw4bit_step(h["p"], h["g"], h["mc"], h["vc"], h["ms"], h["vs"], qm, qv, 0.9, 0.999, 1e-3, 0.01, 1e-8, 3.0)
        assert assert_codes(to_np(d["mc"]), h["mc"], n, f"m codes of tensor {i}") == 0
        assert assert_codes(to_np(d["vc"]), h["vc"], n, f"v codes of tensor {i}") == 0
        np.testing.assert_array_equal(to_np(d["ms"]), h["ms"])
        np.testing.assert_array_equal(to_np(d["vs"]), h["vs"])
        assert_params(to_np(d["p"]), h["p"], p_before, f"p of tensor {i}")


def test_fused_step_extreme_scales(oracle, qmaps):
    """Group maxima outside [2^-60, 2^60] leave the reciprocal-based division for the plain one;
    gradients small enough that g*g underflows give all-zero v groups (code 15, scale 0)."""
    for scale in (1e-12, 1e-22, 1e12, 3e-10):
        def grad_fn(rng, n, s, scale=scale):
            g = (rng.standard_normal(n) * scale).astype(np.float32)
            g[:128] *= 1e-6
            return g

        _run_fused_steps(oracle, qmaps, 128 * 40 + 30, steps=3, seed=int(abs(np.log10(scale))), grad_fn=grad_fn)


def test_fused_step_other_maps(oracle):
    """Maps other than the two standard ones take the generic search in the same kernel:
    a signed linear map for m (create_pow_map(4, True, 1)) and a quadratic map for v."""
    qm = oracle.create_pow_map(4, True, 1)
    qv = (oracle.qmap_v() ** 2).astype(np.float32)
    _run_fused_steps(oracle, (qm, qv), 128 * 300 + 64, steps=4, seed=77)
    # one standard, one not
    _run_fused_steps(oracle, (oracle.qmap_m(), qv), 128 * 50, steps=3, seed=78)
    _run_fused_steps(oracle, (qm, oracle.qmap_v()), 128 * 50, steps=3, seed=79)


def test_near_exact_arithmetic_selftest():
    """sqrt_fast / div_fast (parameter update only) against the correctly rounded device
    operations on every 16th positive normal float and 2^30 divisor pairs; the reciprocal-based
    group division, which decides codes, must agree with IEEE division on every pair, and the
    Newton-corrected reciprocal it starts from with 1/y on every float of its range."""
    lib = _native().lib()
    counts = torch.zeros(11, dtype=torch.int64, device="cuda")
    st = lib.lpmm_selftest_arithmetic(counts.data_ptr(), 16, 1 << 30, 12345, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    c = counts.cpu().tolist()
    print("sqrt: %d tried, %d differ, %d by > 1 ulp, %d at x >= 2^-100; div: %d tried, %d differ, %d by > 1 ulp; "
          "group div: %d tried, %d differ; reciprocal: %d tried, %d differ" % tuple(c))
    assert c[0] > 1.3e8 and c[4] >= 1 << 30 and c[7] >= 1 << 30
    assert c[2] == 0 and c[3] == 0   # sqrt: never more than 1 ulp, exact from 2^-100 upwards
    assert c[5] == 0 and c[6] == 0   # division for the update: exact on this sample
    assert c[8] == 0                 # division by the group maximum: exact
    assert c[9] == 0x5d800000 - 0x21800000 + 1 and c[10] == 0   # its reciprocal: exact on the whole range


def test_device_encoders_exhaustive():
    """The code assignment as the kernels run it on the device (LDS encode table + median-of-three
    clamp for m; fma + ceil + saturating byte conversion + byte permute for v; the division by
    the group maximum in front of both) against the count of midpoints below x, i.e. the
    reference search (lpmm/cpp_extension/fused_adamw_kernel.cu:27-49): all 2^32 bit patterns
    through both maps, NaN -> 15 included, and 256 group maxima around and outside the range
    that divides by the corrected reciprocal."""
    lib = _native().lib()
    counts = torch.zeros(10, dtype=torch.int64, device="cuda")
    st = lib.lpmm_selftest_encoders(counts.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    c = counts.cpu().tolist()
    print("m: %d tried, %d wrong; v: %d tried, %d wrong; bare v form: %d tried, %d wrong; "
          "scaled m: %d tried, %d wrong; scaled v: %d tried, %d wrong" % tuple(c))
    assert c[0] == 1 << 32 and c[2] == 1 << 32
    # the bare form is tried on whole groups of 8 consecutive patterns that are all <= 1.0: the
    # finite negative values and [+0, 1.0) (1.0 and -inf share their groups with values above 1.0
    # and NaNs; they go through the guarded form above)
    assert c[4] == (0xff800000 - 0x80000000) + 0x3f800000
    assert c[6] == 256 * (1 << 16) * 8 and c[8] == c[6]
    assert c[1] == 0 and c[3] == 0 and c[5] == 0 and c[7] == 0 and c[9] == 0


def test_fused_multi_step_under_graph_capture(qmaps):
    """The library only enqueues kernels on the stream it is given (no allocation, no memset, no
    synchronisation), so a multi-tensor step can be recorded into a HIP graph.  Each of three
    replays, with eager work and synchronisations in between, must leave exactly what the same
    call leaves when it is issued eagerly on copies of the buffers."""
    nat = _native()
    lib = nat.lib()
    dqm, dqv = to_dev(qmaps[0]), to_dev(qmaps[1])
    gen = torch.Generator(device="cuda").manual_seed(8)
    sizes = [2048 * 40, 128 * 1001 + 64, 4098, 2048 * 7]

    def make():
        ts = []
        for n in sizes:
            ts.append(dict(n=n, p=torch.randn(n, device="cuda", generator=gen) * 0.02,
                           g=torch.randn(n, device="cuda", generator=gen) * 1e-3,
                           mc=torch.zeros((n + 1) // 2, dtype=torch.uint8, device="cuda"),
                           vc=torch.zeros((n + 1) // 2, dtype=torch.uint8, device="cuda"),
                           ms=torch.zeros((n + 127) // 128, device="cuda"),
                           vs=torch.zeros((n + 127) // 128, device="cuda")))
        return ts

    captured = make()
    eager = [{k: (v.clone() if torch.is_tensor(v) else v) for k, v in t.items()} for t in captured]

    def table(ts):
        return np.array([(t["p"].data_ptr(), t["g"].data_ptr(), t["mc"].data_ptr(), t["vc"].data_ptr(),
                          t["ms"].data_ptr(), t["vs"].data_ptr(), t["n"], 3.0, 0.0) for t in ts],
                        dtype=nat.ADAMW4BIT_TENSOR)

    def enqueue(ts):
        tb = table(ts)
        st = lib.lpmm_adamw4bit_step_multi(tb.ctypes.data, len(ts), dqm.data_ptr(), dqv.data_ptr(), HYPER["beta1"],
                                           HYPER["beta2"], HYPER["lr"], HYPER["wd"], HYPER["eps"],
                                           torch.cuda.current_stream().cuda_stream)
        assert st == 0, lib.lpmm_status_string(st)

    side = torch.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            enqueue(captured)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    # capture records, it does not run: the buffers are untouched so far
    assert all(torch.equal(c["p"], e["p"]) and int(c["mc"].max()) == 0 for c, e in zip(captured, eager))
    for replay in range(3):
        graph.replay()
        enqueue(eager)
        scratch = torch.randn(1 << 16, device="cuda", generator=gen).sum()  # unrelated eager work between replays
        torch.cuda.synchronize()
        assert torch.isfinite(scratch)
        for c, e in zip(captured, eager):
            for k in ("p", "mc", "vc", "ms", "vs"):
                assert torch.equal(c[k], e[k]), f"{k} of the {c['n']}-element tensor differs on replay {replay}"
        for c in captured:  # new gradients for the next replay, written into the captured buffers
            c["g"].copy_(torch.randn(c["n"], device="cuda", generator=gen) * 1e-3)
        for c, e in zip(captured, eager):
            e["g"].copy_(c["g"])
