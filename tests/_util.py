import torch

TOL = 2e-2  # parity bar: max|out - ref| <= TOL * max|ref| after rounding both to the output dtype


def rel_err(out: torch.Tensor, ref: torch.Tensor) -> float:
    a, b = out.detach().float().cpu(), ref.detach().float().cpu()
    assert a.shape == b.shape, (a.shape, b.shape)
    assert torch.equal(torch.isnan(a), torch.isnan(b)), "NaN pattern differs"
    a, b = torch.nan_to_num(a), torch.nan_to_num(b)
    denom = b.abs().max().item()
    return ((a - b).abs().max().item() / denom) if denom > 0 else (a - b).abs().max().item()
