"""Host-side behaviour that needs no GPU: the C ABI's symbols and argument checks, the
config reader, the optimizer's state bookkeeping and error behaviour."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
HEADER = os.path.join(ROOT, "include", "lpmm_hip.h")


def declared_functions():
    txt = open(HEADER).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(lpmm_[a-z0-9_]+)\s*\(", txt)))


def test_library_exports_every_declared_symbol():
    from lpmm import _native

    lib = ctypes.CDLL(_native.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 17
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/lpmm_hip.h but not exported"
    assert sorted(_native.PROTOTYPES) == names, "lpmm/_native.py prototypes differ from the header"
    assert _native.lib().lpmm_abi_version() == _native.ABI_VERSION


def test_record_layouts_match_header():
    from lpmm import _native

    assert _native.ADAMW4BIT_TENSOR.itemsize == 64 and _native.ADAMW_FP32_TENSOR.itemsize == 48
    assert _native.ADAMW4BIT_TENSOR.fields["n"][1] == 48 and _native.ADAMW4BIT_TENSOR.fields["step"][1] == 56
    assert _native.ADAMW_FP32_TENSOR.fields["n"][1] == 32 and _native.ADAMW_FP32_TENSOR.fields["step"][1] == 40
    assert _native.NONFUSED_RANK1_F16_TENSOR.itemsize == 104 and _native.NONFUSED_RANK1_F16_TENSOR.fields["work"][1] == 72
    assert _native.NONFUSED_RANK1_F16_TENSOR.fields["rows"][1] == 80 and _native.NONFUSED_RANK1_F16_TENSOR.fields["step"][1] == 96
    header = open(os.path.join(ROOT, "include", "lpmm_hip.h")).read()
    assert int(re.search(r"#define LPMM_MULTI_MAX (\d+)", header).group(1)) == _native.MULTI_MAX


def test_argument_errors_without_gpu():
    """Validation precedes any HIP call: NULL, misaligned and out-of-range arguments are
    reported as status codes on a machine without a GPU."""
    from lpmm import _native

    lib = _native.lib()
    buf = np.zeros(64, np.float32)
    ptr = buf.ctypes.data
    NULL, ALIGN, SIZE = 1, 2, 3
    f6 = (0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0)
    assert lib.lpmm_adamw4bit_step(None, ptr, ptr, ptr, ptr, ptr, ptr, ptr, 16, *f6, None) == NULL
    assert lib.lpmm_adamw4bit_step(ptr, ptr, ptr, ptr, ptr, ptr, None, ptr, 16, *f6, None) == NULL
    assert lib.lpmm_adamw4bit_step(ptr + 2, ptr, ptr, ptr, ptr, ptr, ptr, ptr, 16, *f6, None) == ALIGN
    assert lib.lpmm_adamw4bit_step(ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, -1, *f6, None) == SIZE
    assert lib.lpmm_adamw4bit_step(ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, 0, *f6, None) == 0  # nothing to do
    assert lib.lpmm_adamw4bit_step_multi(None, 3, ptr, ptr, *f6[:5], None) == NULL
    assert lib.lpmm_adamw4bit_step_multi(None, 0, ptr, ptr, *f6[:5], None) == 0
    assert lib.lpmm_adamw_fp32_step(ptr, None, ptr, ptr, 16, *f6, None) == NULL
    assert lib.lpmm_pack_nonlinear_4bit(ptr, ptr, 12, ptr, None) == SIZE  # not a multiple of 8
    assert lib.lpmm_pack_nonlinear_4bit(None, ptr, 16, ptr, None) == NULL
    assert lib.lpmm_unpack_nonlinear_4bit(ptr, ptr, -5, ptr, None) == SIZE
    assert lib.lpmm_quant_group(ptr, 64, 100, ptr, ptr, ptr, None) == SIZE  # group size not 128 * 2^k
    assert lib.lpmm_quant_group(ptr, 64, 8192, ptr, ptr, ptr, None) == SIZE
    assert lib.lpmm_quant_group(ptr, 0, 128, ptr, ptr, ptr, None) == SIZE
    assert lib.lpmm_dequant_group(ptr, ptr, ptr, 64, 64, ptr, None) == SIZE
    assert lib.lpmm_rank1_stats(ptr, 0, 8, ptr, ptr, None) == SIZE
    assert lib.lpmm_quant_rank1(ptr, 8, 8, None, ptr, ptr, ptr, None) == NULL
    assert lib.lpmm_dequant_rank1(ptr, ptr, ptr, ptr, 8, -8, ptr, None) == SIZE
    assert lib.lpmm_nonfused_update(ptr, ptr, ptr + 1, ptr, 16, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0, None) == ALIGN
    assert lib.lpmm_factored_stats(ptr, 8, 8, ptr, ptr, ptr, 0.999, None, None) == NULL
    assert lib.lpmm_factored_update(ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, 0, 8, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0,
                                    0, None) == SIZE
    # 64 x 256 tiles: 64 row tiles of column partials, 43 column tiles of row partials, 16 row-block sums, the mean
    assert lib.lpmm_factored_workspace_bytes(4096, 11008) == (64 * 11008 + 43 * 4096 + 16 + 1) * 8
    assert lib.lpmm_status_string(NULL).decode().startswith("a required pointer")
    with pytest.raises(RuntimeError, match="status 3"):
        _native.check(SIZE, "probe")


def test_config_defaults_and_yaml():
    from lpmm.config import CONFIG_DIR, get_config

    c = get_config(None)
    # built-in default for v is 'group', not 'rank1' (lpmm/config.py:58); README's default.yml says rank1
    assert c.QUANT.SQM.SCALE_TYPE.DEFAULT == "group" and c.QUANT.M.SCALE_TYPE.DEFAULT == "group"
    assert c.QUANT.M.BITS == 4 and c.QUANT.M.SIGNED is True and c.QUANT.M.QUANT_TYPE.DEFAULT == "nonlinear"
    assert c.QUANT.SQM.SIGNED is False and c.QUANT.SQM.QUANT_TYPE.DEFAULT == "power-1"
    assert c.QUANT.M.THRESHOLD == 4096 and c.QUANT.M.ROUND_TYPE == "real-nearest" and c.QUANT.M.GROUP_SIZE == 128
    d = get_config(os.path.join(CONFIG_DIR, "default.yml"))
    assert d.QUANT.SQM.SCALE_TYPE.DEFAULT == "rank1" and d.QUANT.SQM.SIGNED is False  # untouched keys survive
    assert get_config(os.path.join(CONFIG_DIR, "2nd_moment_group_128.yml")).QUANT.SQM.SCALE_TYPE.DEFAULT == "group"
    assert get_config(os.path.join(CONFIG_DIR, "1st_moment_group_512.yml")).QUANT.M.GROUP_SIZE == 512
    assert get_config(os.path.join(CONFIG_DIR, "2nd_moment_only_default.yml")).QUANT.M.ENABLE is False
    assert get_config(None).QUANT.SQM.SCALE_TYPE.DEFAULT == "group"  # defaults are not mutated by merges
    with pytest.raises(TypeError):
        get_config(42)


def test_config_base_inheritance(tmp_path):
    from lpmm.config import get_config

    (tmp_path / "base.yml").write_text("QUANT:\n  M:\n    GROUP_SIZE: 256\n  SQM:\n    THRESHOLD: 100\n")
    (tmp_path / "child.yml").write_text("BASE: ['base.yml']\nQUANT:\n  SQM:\n    SCALE_TYPE: {DEFAULT: rank1}\n")
    c = get_config(str(tmp_path / "child.yml"))
    assert c.QUANT.M.GROUP_SIZE == 256 and c.QUANT.SQM.THRESHOLD == 100 and c.QUANT.SQM.SCALE_TYPE.DEFAULT == "rank1"


def test_optimizer_argument_validation():
    import lpmm

    p = [torch.nn.Parameter(torch.zeros(4))]
    for kw in (dict(lr=-1.0), dict(eps=-1e-8), dict(betas=(1.0, 0.999)), dict(betas=(0.9, -0.1)), dict(weight_decay=-1)):
        with pytest.raises(ValueError):
            lpmm.optim.AdamW(p, **kw)
    opt = lpmm.optim.AdamW(p, lr=1e-3, fused=True, factor_second_moment=True)
    g = opt.param_groups[0]
    assert g["fused"] is True and g["factor_second_moment"] is True and g["use_first_moment"] is True
    assert g["betas"] == (0.9, 0.999) and g["eps"] == 1e-8 and g["weight_decay"] == 1e-2
    with pytest.raises(ValueError):
        opt.get_subqconfig("nope")
    md = opt.get_qmetadata_by_state_name("exp_avg")
    assert md == dict(b=4, scale_type="group", quant_type="nonlinear", round_type="real-nearest", gp_sz=128, signed=True)
    md = opt.get_qmetadata_by_state_name("exp_avg_sq")
    assert md == dict(b=4, scale_type="group", quant_type="power-1", round_type="real-nearest", gp_sz=128, signed=False)


def test_sgd_argument_validation():
    import lpmm

    p = [torch.nn.Parameter(torch.zeros(4))]
    for kw in (dict(lr=-1.0), dict(lr=0.1, momentum=-0.5), dict(lr=0.1, weight_decay=-1.0), dict(lr=0.1, fused=True)):
        with pytest.raises(ValueError):
            lpmm.optim.SGD(p, **kw)
    opt = lpmm.optim.SGD(p, lr=0.1, momentum=0.9)
    assert opt.get_qmetadata_by_state_name("momentum_buffer")["quant_type"] == "nonlinear"
    with pytest.raises(ValueError):
        opt.get_subqconfig("exp_avg")


def test_state_init_threshold_and_override():
    """State layout on first use (lpmm/optim/adamw.py:114-129) and the numel > 4096 rule
    (lpmm/optim/optimizer.py:156-163); needs no GPU because only the bookkeeping runs."""
    import lpmm

    big = torch.nn.Parameter(torch.zeros(64, 65))     # 4160 > 4096
    edge = torch.nn.Parameter(torch.zeros(64, 64))    # 4096: not quantised
    forced = torch.nn.Parameter(torch.zeros(100, 100))
    holder = torch.nn.Module()
    holder.w = forced
    opt = lpmm.optim.AdamW([big, edge, forced], factor_second_moment=False)
    opt.override_quantize_enable(holder, "w", False)
    group = opt.param_groups[0]
    for p in (big, edge, forced):
        state, factored = opt._state_of(group, p)
        assert not factored
        assert set(state) == {"step", "exp_avg", "exp_avg_sq", "exp_avg_qstate", "exp_avg_sq_qstate"}
        assert state["step"].device.type == "cpu" and float(state["step"]) == 0.0
        assert state["exp_avg"].dim() == 0 and state["exp_avg_sq"].dim() == 0
        assert set(state["exp_avg_qstate"]) == {"enable", "overhead", "qmap"}
        assert state["exp_avg_qstate"]["qmap"].numel() == 16
    assert opt.state[big]["exp_avg_qstate"]["enable"] is True
    assert opt.state[edge]["exp_avg_qstate"]["enable"] is False
    assert opt._enabled(forced, opt.state[forced], "exp_avg") is False
    assert opt.state[big]["exp_avg_qstate"]["qmap"] is opt.state[forced]["exp_avg_qstate"]["qmap"]  # cached
    with pytest.raises(ValueError):
        opt.override_quantize_enable(holder, "w", True)  # state already exists
    fopt = lpmm.optim.AdamW([torch.nn.Parameter(torch.zeros(3, 8, 16))], factor_second_moment=True)
    p = fopt.param_groups[0]["params"][0]
    state, factored = fopt._state_of(fopt.param_groups[0], p)
    assert factored and state["exp_avg_sq_row"].shape == (3, 8) and state["exp_avg_sq_col"].shape == (3, 16)
    assert "exp_avg_sq" not in state


def test_cpu_tensors_are_rejected_loudly():
    """There is no CPU path: a step on CPU parameters raises like the reference's operators
    (lpmm/cpp_extension/common.h:15-27)."""
    import lpmm
    from lpmm.cpp_extension import fused_adamw, quantization

    p = torch.nn.Parameter(torch.randn(100, 100))
    p.grad = torch.randn(100, 100)
    for fused in (True, False):
        opt = lpmm.optim.AdamW([p], fused=fused)
        with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
            opt.step()
    z = torch.zeros(8)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        fused_adamw.adamw_single_tensor(z, z, z, z, 0.9, 0.999, 1e-3, 0.01, 1e-8, 1.0)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        quantization.pack_nonlinear(torch.zeros(1, 8), torch.zeros(16), 4, False)
    with pytest.raises(RuntimeError):
        quantization.pack_nonlinear(torch.zeros(1, 8), torch.zeros(16), 9, False)  # bits <= 8
    sparse = torch.nn.Parameter(torch.randn(10, 10))
    sparse.grad = torch.randn(10, 10).to_sparse()
    with pytest.raises(RuntimeError, match="sparse"):
        lpmm.optim.AdamW([sparse]).step()


def test_state_dict_round_trip_keeps_packed_int8():
    """load_state_dict moves state to the parameter's device/dtype but never converts the
    packed int8 tensors or `step` (lpmm/optim/optimizer.py:95-115)."""
    import lpmm

    p = torch.nn.Parameter(torch.zeros(64, 65, dtype=torch.float64))
    opt = lpmm.optim.AdamW([p], fused=True)
    state, _ = opt._state_of(opt.param_groups[0], p)
    state["step"] += 3
    state["exp_avg"] = torch.arange(-100, 100, dtype=torch.int8)
    state["exp_avg_sq"] = torch.arange(0, 120, dtype=torch.int8)
    state["exp_avg_qstate"]["overhead"]["max1"] = torch.rand(33)
    state["exp_avg_sq_qstate"]["overhead"].update({"max1": None, "max_dims": [torch.rand(64, 1), torch.rand(1, 65)],
                                                   "scaled_shape": torch.Size((64, 65)), "dtype": torch.float32,
                                                   "stride": (65, 1), "dim": 2})
    sd = opt.state_dict()
    assert "qconfig" in sd
    opt2 = lpmm.optim.AdamW([torch.nn.Parameter(torch.zeros(64, 65, dtype=torch.float64))], fused=True)
    opt2.load_state_dict(sd)
    s2 = opt2.state[opt2.param_groups[0]["params"][0]]
    assert s2["exp_avg"].dtype == torch.int8 and torch.equal(s2["exp_avg"], state["exp_avg"])
    assert s2["exp_avg_sq"].dtype == torch.int8
    assert float(s2["step"]) == 3.0 and s2["step"].dtype == torch.float32
    assert s2["exp_avg_qstate"]["overhead"]["max1"].dtype == torch.float64  # float state follows the parameter
    # ... except the maps: the kernels read them as floats, and a rounded map would decode the codes differently
    assert s2["exp_avg_qstate"]["qmap"].dtype == torch.float32 and s2["exp_avg_sq_qstate"]["qmap"].dtype == torch.float32
    assert torch.equal(s2["exp_avg_qstate"]["qmap"], state["exp_avg_qstate"]["qmap"])
    oh = s2["exp_avg_sq_qstate"]["overhead"]
    assert oh["scaled_shape"] == torch.Size((64, 65)) and oh["dtype"] == torch.float32 and oh["dim"] == 2
    assert isinstance(oh["max_dims"], list) and oh["max_dims"][1].shape == (1, 65)
    assert opt2.qconfig.QUANT.M.BITS == 4
    with pytest.raises(ValueError):
        lpmm.optim.AdamW([torch.nn.Parameter(torch.zeros(2)), torch.nn.Parameter(torch.zeros(2))]).load_state_dict(sd)

    # the reference stores its yacs CfgNode under 'qconfig' (lpmm/optim/optimizer.py:68-71): a dict subclass with
    # attribute access, nested in itself.  Any such mapping is accepted and becomes this package's own node type.
    class CfgNodeLike(dict):
        def __getattr__(self, name):
            if name in self:
                return self[name]
            raise AttributeError(name)

    def wrap(value):
        return CfgNodeLike({k: wrap(v) for k, v in value.items()}) if isinstance(value, dict) else value

    sd3 = dict(sd, qconfig=wrap(sd["qconfig"]))
    sd3["qconfig"]["QUANT"]["SQM"]["SCALE_TYPE"]["DEFAULT"] = "rank1"
    opt3 = lpmm.optim.AdamW([torch.nn.Parameter(torch.zeros(64, 65, dtype=torch.float64))], fused=True)
    opt3.load_state_dict(sd3)
    assert type(opt3.qconfig) is lpmm.config.Node and type(opt3.qconfig.QUANT.SQM) is lpmm.config.Node
    assert opt3.qconfig.QUANT.SQM.SCALE_TYPE.DEFAULT == "rank1"
    assert type(opt3.state_dict()["qconfig"]) is dict
    with pytest.raises(ValueError, match="lacks QUANT.M"):
        opt3.load_state_dict(dict(sd, qconfig={"QUANT": {"SQM": sd["qconfig"]["QUANT"]["SQM"]}}))


def test_oracle_under_sanitizers(tmp_path):
    """The oracle's C code under AddressSanitizer + UBSan on ragged sizes (host only)."""
    exe = str(tmp_path / "oracle_sanitize")
    subprocess.check_call(["gcc", "-O1", "-g", "-std=c11", "-ffp-contract=off", "-fsanitize=address,undefined",
                           "-fno-sanitize-recover=all", "-fno-omit-frame-pointer", "-static-libasan",
                           os.path.join(HERE, "oracle_sanitize_driver.c"), os.path.join(ROOT, "oracle", "lpmm_oracle.c"),
                           "-lm", "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stderr[-2000:]
    assert "ok" in out.stdout


def test_utils_metrics_and_bookkeeping():
    """lpmm.utils: closed forms of the error metrics, byte counting, rank helpers."""
    from lpmm import utils

    x = torch.tensor([3.0, 4.0])
    qx = torch.tensor([3.0, 3.0])
    assert utils.relerr(x, qx).item() == pytest.approx(1.0 / 5.0)
    assert utils.abserr(x, qx).item() == pytest.approx(0.5)
    assert utils.sqnr(x, qx).item() == pytest.approx(20 * np.log10(5.0), rel=1e-6)
    assert utils.compute_tensor_bytes([torch.zeros(10), torch.zeros(6, dtype=torch.int8),
                                       torch.zeros(4, dtype=torch.bfloat16)]) == 40 + 6 + 8
    assert utils.compute_tensor_bytes(torch.zeros(3, dtype=torch.float64)) == 0  # a type the reference does not list
    assert utils.get_rank() == 0 and utils.get_world_size() == 1
    assert utils.get_metric_fn("min")(1, 2) and utils.get_metric_fn("max")(2, 1)
    with pytest.raises(NotImplementedError):
        utils.get_metric_fn("median")


def test_every_shipped_configuration_merges_to_the_reference_settings():
    """The 13 files under lpmm/configs carry the reference's names; merged over the defaults each
    must give the settings of the reference's file of that name (lpmm/configs/*.yml there):
    (m enabled, m bits, m block size, v bits, v scale type)."""
    import lpmm
    from lpmm.config import get_config

    want = {
        "default.yml": (True, 4, 128, 4, "rank1"),
        "default_5b.yml": (True, 5, 128, 5, "rank1"),
        "default_6b.yml": (True, 6, 128, 6, "rank1"),
        "default_7b.yml": (True, 7, 128, 7, "rank1"),
        "default_8b.yml": (True, 8, 128, 8, "rank1"),
        "1st_moment_group_256.yml": (True, 4, 256, 4, "rank1"),
        "1st_moment_group_512.yml": (True, 4, 512, 4, "rank1"),
        "1st_moment_group_1024.yml": (True, 4, 1024, 4, "rank1"),
        "1st_moment_group_2048.yml": (True, 4, 2048, 4, "rank1"),
        "1st_moment_group_4096.yml": (True, 4, 4096, 4, "rank1"),
        "2nd_moment_group_128.yml": (True, 4, 128, 4, "group"),
        "2nd_moment_only_default.yml": (False, 4, 128, 4, "rank1"),
        "2nd_moment_only_group_128.yml": (False, 4, 128, 4, "group"),
    }
    cfg_dir = os.path.join(os.path.dirname(lpmm.config.__file__), "configs")
    assert sorted(os.listdir(cfg_dir)) == sorted(want)
    for name, (m_on, m_bits, m_gp, v_bits, v_scale) in want.items():
        q = get_config(os.path.join(cfg_dir, name)).QUANT
        got = (q.M.ENABLE, q.M.BITS, q.M.GROUP_SIZE, q.SQM.BITS, q.SQM.SCALE_TYPE.DEFAULT)
        assert got == (m_on, m_bits, m_gp, v_bits, v_scale), name
        # everything else stays at the defaults the two files share
        assert q.SQM.ENABLE is True and q.SQM.GROUP_SIZE == 128 and q.M.SCALE_TYPE.DEFAULT == "group"
        assert q.M.QUANT_TYPE.DEFAULT == "nonlinear" and q.SQM.QUANT_TYPE.DEFAULT == "power-1"
        assert q.M.ROUND_TYPE == "real-nearest" and q.SQM.ROUND_TYPE == "real-nearest"
        assert q.M.SIGNED is True and q.SQM.SIGNED is False and q.M.THRESHOLD == 4096
