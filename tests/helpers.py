"""Synthetic inputs of the benchmark configurations and the comparison rules shared by the GPU parity tests."""
import numpy as np
import torch

from oracle import ksq_oracle as orc

F16, BF16 = 0, 1
TORCH_DT = {F16: torch.float16, BF16: torch.bfloat16}


def gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def bits_of(t):
    """torch 16-bit float tensor (cpu) -> numpy uint16 bit patterns."""
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def uniform(g, shape, lo, hi, dtype):
    return (torch.rand(shape, generator=g) * (hi - lo) + lo).to(TORCH_DT[dtype])


def make_w4a16(seed, M, N, K, group, dtype, awq, x_std=1.0, s_lo=0.004, s_hi=0.02, z_lo=6, z_hi=9):
    """Returns a dict with checkpoint-format tensors (torch, cpu) and the numpy views the oracle needs."""
    g = gen(seed)
    codes = torch.randint(0, 16, (K, N), generator=g, dtype=torch.uint8)
    scales = uniform(g, (K // group, N), s_lo, s_hi, dtype)
    x = (torch.randn((M, K), generator=g) * x_std).to(TORCH_DT[dtype])
    d = {"codes": codes.numpy(), "scales": scales, "x": x, "M": M, "N": N, "K": K, "group": group, "dtype": dtype}
    if awq:
        zeros = torch.randint(z_lo, z_hi + 1, (K // group, N), generator=g, dtype=torch.uint8)
        d["zeros"] = zeros.numpy()
        d["qweight"] = torch.from_numpy(orc.awq_pack(d["codes"]).view(np.int32))
        d["qzeros"] = torch.from_numpy(orc.awq_pack(d["zeros"]).view(np.int32))
    else:
        d["zeros"] = None
        d["qweight"] = torch.from_numpy(orc.gptq_pack(d["codes"]).view(np.int32))
    return d


def w4a16_oracle(d):
    return orc.w4a16_gemm(bits_of(d["x"]), d["codes"], bits_of(d["scales"]), d["zeros"], d["group"], d["dtype"])


def ulp(ref, dtype):
    """Spacing of the output type at |ref| (fp16: 10 mantissa bits, bf16: 7)."""
    mant = 10 if dtype == F16 else 7
    a = np.maximum(np.abs(ref.astype(np.float64)), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(a)) - mant)


def check_gemm(y_gpu, ref_f32, dtype, what="", weights_rounded=False, rel_l2_max=5e-3):
    """rel-L2 <= 5e-3 and max-abs <= 2e-2 against the fp32-accumulated dequant reference.

    Two forms of the absolute bound are used and the raw maximum is returned for reporting:
      * every kernel: max|y - ref| / max(1, max|ref|) <= 2e-2;
      * kernels that keep the weights exact inside the MFMA (split-K decode, fp8, MoE decode): the error left after
        allowing for the output type's own rounding (half a unit in the last place of the reference value) must stay
        below 2e-2 in absolute terms.  Once |y| >= 8 in bf16 half an ulp alone is 0.031, so the raw difference cannot
        meet 2e-2 for any kernel.
    The prefill kernel rounds every dequantized weight to T before the MFMA, as the reference's Marlin and Triton
    kernels do; with bf16's 8-bit mantissa that rounding alone adds a few 1e-3 * |y| and only the first form applies
    (weights_rounded=True).
    """
    y = y_gpu.float().cpu().numpy().astype(np.float64)
    ref = ref_f32.astype(np.float64)
    assert y.shape == ref.shape
    assert np.all(np.isfinite(y)), what
    rel_l2 = np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30)
    err = np.abs(y - ref)
    assert rel_l2 <= rel_l2_max, "%s rel-L2 %.3e" % (what, rel_l2)
    norm = err.max() / max(1.0, np.abs(ref).max())
    assert norm <= 2e-2, "%s normalised max-abs %.3e (raw %.3e)" % (what, norm, err.max())
    if not weights_rounded:
        excess = np.maximum(err - 0.5 * ulp(ref, dtype), 0.0).max()
        assert excess <= 2e-2, "%s max-abs beyond output rounding %.3e (raw %.3e)" % (what, excess, err.max())
    return rel_l2, err.max()


def check_gemm_f32(y32_gpu, ref_f32, what=""):
    """The parity bar as it is written, on the sums before they are rounded to the output type (the fp32 entry points):
    rel-L2 <= 5e-3 and max-abs <= 2e-2 against the fp32-accumulated dequant reference, raw, nothing normalised."""
    y = y32_gpu.cpu().numpy().astype(np.float64)
    ref = ref_f32.astype(np.float64)
    assert y.shape == ref.shape and np.all(np.isfinite(y)), what
    rel_l2 = np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30)
    max_abs = np.abs(y - ref).max()
    assert rel_l2 <= 5e-3, "%s rel-L2 before rounding %.3e" % (what, rel_l2)
    assert max_abs <= 2e-2, "%s max-abs before rounding %.3e" % (what, max_abs)
    return rel_l2, max_abs


def each_regime(m):
    """Once as the library decides by default and, for more than 32 rows, once more with the small-problem rule off
    (every such problem on the MFMA tile kernels): `for rule in each_regime(m): ...` runs the body under each setting.
    conftest restores the default after the test whatever happens inside the loop."""
    from ksanallm_amd import lib as L

    for rule in ((True, False) if m > 32 else (True,)):
        L.set_small_problem_rule(rule)
        yield rule
    L.set_small_problem_rule(True)
