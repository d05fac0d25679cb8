"""Comparison helpers with the error measure of the reference (testing.py:21-80):
every element's error is taken relative to max(|ref|, rms(ref)); both the maximum
and the RMS of that relative error are bounded."""
import torch


def assert_equal(ref, tri):
    if isinstance(ref, torch.Tensor):
        assert torch.equal(ref.cpu(), tri.cpu()), f"tensors differ:\n{ref}\nvs\n{tri}"
    else:
        assert ref == tri, f"{ref} != {tri}"


def relative_errors(ref: torch.Tensor, tri: torch.Tensor):
    """(max, rms) of |ref - tri| / max(|ref|, rms(ref)); matching infinities count as equal."""
    ref = ref.detach().to(torch.float32).cpu()
    tri = tri.detach().to(torch.float32).cpu()
    assert ref.shape == tri.shape, f"Tensors must have same size {ref.shape=} {tri.shape=}"
    inf_r, inf_t = torch.isinf(ref), torch.isinf(tri)
    assert torch.equal(inf_r, inf_t), "Tensor must have same infinite elements"
    r = torch.where(inf_r, torch.zeros_like(ref), ref)
    t = torch.where(inf_t, torch.zeros_like(tri), tri)
    norm = 1.0 / (r.abs().max() + 1e-30)  # keeps the squares finite
    r, t = r * norm, t * norm
    floor = torch.sqrt((r * r).mean()) + 1e-30
    rel = (r - t).abs() / torch.maximum(floor, r.abs())
    return float(rel.max()), float(torch.sqrt((rel * rel).mean()))


def assert_close(ref, tri, maxtol=None, rmstol=None, description="--", verbose=True):
    """Defaults: maximum relative error 2e-2, RMS relative error 4e-3."""
    if tri.dtype.itemsize == 1:
        cast = ref.to(tri.dtype)
        if ref.dtype == tri.dtype:
            assert torch.equal(cast.view(torch.uint8).cpu(), tri.view(torch.uint8).cpu())
            return
        ref = cast
    if ref.numel() == 0:
        return
    maxtol = 2e-2 if maxtol is None else maxtol
    rmstol = 4e-3 if rmstol is None else rmstol
    max_err, rms_err = relative_errors(ref, tri)
    if verbose:
        print(f"{description} maximum relative error = {max_err} (threshold = {maxtol})")
        print(f"{description} RMS relative error = {rms_err} (threshold = {rmstol})")
    assert max_err <= maxtol, f"{description}: maximum relative error {max_err} > {maxtol}"
    assert rms_err <= rmstol, f"{description}: RMS relative error {rms_err} > {rmstol}"
