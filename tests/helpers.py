"""Shared helpers of the parity tests."""
import torch


def bits(t: torch.Tensor) -> torch.Tensor:
    """Raw storage bits (so that -0.0 != 0.0 and NaNs compare by pattern)."""
    t = t.detach().cpu().contiguous()
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32)


def ulp_diff(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in representable values of a 16-bit float type (bf16 / fp16)."""
    def key(t):
        i = t.detach().cpu().contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
        return torch.where(i >= 0x8000, 0x8000 - i, i)
    return (key(a) - key(b)).abs()


def assert_parity(got: torch.Tensor, want: torch.Tensor, exact: bool, what: str = "", res=None) -> None:
    """The bar of this repository.

    16-bit storage: at most 1 ulp from the fp32-accumulate oracle (bit exact
    when `exact`).  fp32: bit exact when `exact`, else 1e-5 relative.  When a
    residual term `res` was added, both are taken relative to the larger of
    the result and that term (the sum can cancel, which no evaluation order
    of the SiLU survives).
    """
    got, want = got.detach().cpu(), want.detach().cpu()
    assert got.shape == want.shape and got.dtype == want.dtype, (what, got.shape, want.shape)
    if exact:
        diff = (bits(got) != bits(want)).nonzero()
        first = tuple(diff[0].tolist()) if len(diff) else None
        assert len(diff) == 0, (f"{what}: not bit exact: {len(diff)} of {got.numel()} elements differ, first at {first}: "
                                f"got {got[first].item()!r}, want {want[first].item()!r}")
    elif got.dtype == torch.float32:
        scale = want.abs() if res is None else torch.maximum(want.abs(), res.detach().cpu().float().abs())
        err = (got - want).abs() / scale.clamp_min(1e-3)
        assert err.max().item() <= 1e-5, f"{what}: rel err {err.max().item():.3e} > 1e-5"
    elif res is None:
        d = ulp_diff(got, want)
        assert d.max().item() <= 1, f"{what}: {d.max().item()} ulp > 1"
    else:
        # one unit in the last place of the larger of the result and the residual term
        mant = 7 if got.dtype == torch.bfloat16 else 10
        scale = torch.maximum(want.float().abs(), res.detach().cpu().float().abs()).clamp_min(2.0 ** -14)
        ulp = torch.exp2(torch.floor(torch.log2(scale)) - mant)
        err = (got.float() - want.float()).abs() / ulp
        assert err.max().item() <= 1.0, f"{what}: {err.max().item():.2f} ulp (of the larger term) > 1"


def right_padded_mask(lens, L, dtype=torch.int64):
    m = torch.zeros(len(lens), L, dtype=dtype)
    for b, n in enumerate(lens):
        m[b, :n] = 1
    return m
