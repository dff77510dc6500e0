"""Shared helpers of the test-suite (oracle <-> torch glue, error metrics)."""
import numpy as np
import torch

import oracle as O


def t2bits(t):
    """bf16 torch tensor -> numpy uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bits2t(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)


def bits2f(a):
    return O.bf16_to_f32(a)


def randn_bf16(shape, std, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)


def block_bf16(W, bk=16, bc=64):
    """torch restatement of the blocked VNNI2 layout (view + permute)."""
    N, K = W.shape
    return W.view(N // bk, bk, K // bc, bc // 2, 2).permute(0, 2, 3, 1, 4).contiguous()


def err_stats(got_bits, ref_bits):
    g = bits2f(got_bits).astype(np.float64)
    r = bits2f(ref_bits).astype(np.float64)
    d = np.abs(g - r)
    rms = float(np.sqrt(np.mean(r * r))) or 1.0
    return {
        "max_abs": float(d.max()),
        "rel_l2": float(np.sqrt((d * d).sum()) / (np.sqrt((r * r).sum()) or 1.0)),
        "mismatch_frac": float(np.mean(got_bits != ref_bits)),
        "rms": rms,
        "viol": d - (2.0 ** -7 * np.abs(r) + 2.0 ** -8 * rms),
    }


def assert_close_bf16(got_bits, ref_bits, ulps=1, rel_l2=4e-3, what="", pre_bits=None, max_mismatch="auto"):
    """Tolerance of the parity tests: every element within `ulps` bf16 ulps of
    the oracle (|d| <= ulps * (2^-7 |ref| + 2^-8 rms(ref)), the second term
    covering outputs that cancel to near zero) and relative L2 error <= rel_l2.
    `max_mismatch` bounds how many elements may differ from the oracle's bits AT
    ALL: a different fp32 summation order moves 5-100 elements per million
    across a rounding boundary, so a kernel that is one ulp off everywhere is an
    error even though each element is within the bound.  "auto" = 1e-3 of the
    elements (at least 3) for the 1-ulp comparisons, no count for the 2-ulp ones
    (SiLU / GELU go through the hardware's exp2 and reciprocal, whose results
    differ from libm's in more places).
    `pre_bits` = the oracle's bf16 GEMM(+bias) tile before an additive post-op.
    A different fp32 summation order moves a few elements per million of that
    tile by one bf16 ulp (the no-post tests accept exactly that); the post-op
    then rounds pre + scale*in once more on each side, and when both sums fall
    on a rounding tie the two results end up ulp(pre) + ulp(out) apart. So one
    exact ulp of the pre value is added to the bound."""
    s = err_stats(got_bits, ref_bits)
    g = bits2f(got_bits).astype(np.float64)
    r = bits2f(ref_bits).astype(np.float64)
    bound = ulps * (2.0 ** -7 * np.abs(r) + 2.0 ** -8 * s["rms"])
    if pre_bits is not None:
        p = np.abs(bits2f(pre_bits).astype(np.float64))
        bound = bound + 2.0 ** (np.floor(np.log2(np.maximum(p, 2.0 ** -126))) - 7)
    bad = np.abs(g - r) > bound
    assert not bad.any(), (
        f"{what}: {int(bad.sum())} elements beyond {ulps} ulp; max_abs={s['max_abs']:.4g} "
        f"rel_l2={s['rel_l2']:.3g} first={np.argwhere(bad)[:4].tolist()}"
    )
    assert s["rel_l2"] <= rel_l2, f"{what}: rel_l2={s['rel_l2']:.3g} > {rel_l2}"
    if max_mismatch == "auto":
        max_mismatch = 1e-3 if ulps == 1 else None
    if max_mismatch is not None:
        n_diff = int(np.count_nonzero(np.asarray(got_bits) != np.asarray(ref_bits)))
        allowed = max(3, int(np.ceil(max_mismatch * np.asarray(ref_bits).size)))
        assert n_diff <= allowed, f"{what}: {n_diff} of {np.asarray(ref_bits).size} elements differ from the oracle (allowed {allowed})"
    return s
