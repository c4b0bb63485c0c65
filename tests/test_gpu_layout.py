"""The modules' layout changes (mpl_transpose behind mplayers_amd.layout) equal
permute().contiguous() bit for bit, forwards and through autograd."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("b,cv,n,h,w", [(1, 1, 192, 37, 53), (2, 1, 21, 65, 65), (1, 2, 7, 1, 300),
                                        (3, 1, 64, 64, 64), (1, 1, 1, 5, 5), (1, 1, 256, 9, 1),
                                        (1, 1, 100, 129, 130)])
def test_layout_matches_permute(gpu, b, cv, n, h, w):
  import torch
  from mplayers_amd import layout
  g = torch.Generator().manual_seed(n + h)
  x = torch.randn(b, cv, n, h, w, generator=g).cuda()
  last = layout.labels_last(x)
  assert last.is_contiguous() and torch.equal(last, x.permute(0, 1, 3, 4, 2).contiguous())
  first = layout.labels_first(last)
  assert first.is_contiguous() and torch.equal(first, x)
  # non-contiguous input, and the gradient path
  y = x.transpose(3, 4)
  assert torch.equal(layout.labels_last(y), y.permute(0, 1, 3, 4, 2).contiguous())
  a = x.clone().requires_grad_(True)
  bref = x.clone().requires_grad_(True)
  wgt = torch.randn(b, cv, h, w, n, generator=g).cuda()
  (layout.labels_last(a) * wgt).sum().backward()
  (bref.permute(0, 1, 3, 4, 2).contiguous() * wgt).sum().backward()
  assert torch.equal(a.grad, bref.grad)
  c = last.clone().requires_grad_(True)
  dref = last.clone().requires_grad_(True)
  wgt2 = torch.randn(b, cv, n, h, w, generator=g).cuda()
  (layout.labels_first(c) * wgt2).sum().backward()
  (dref.permute(0, 1, 4, 2, 3).contiguous() * wgt2).sum().backward()
  assert torch.equal(c.grad, dref.grad)


def test_layout_full_size_and_fallback(gpu):
  import torch
  from mplayers_amd import layout
  x = torch.randn(1, 1, 192, 1500, 2000, device="cuda")
  last = layout.labels_last(x)
  ref = x.permute(0, 1, 3, 4, 2).contiguous()
  assert torch.equal(last, ref)
  del ref
  assert torch.equal(layout.labels_first(last), x)
  # other dtypes take torch's path
  h = torch.randn(1, 1, 4, 5, 6, device="cuda").half()
  assert torch.equal(layout.labels_last(h), h.permute(0, 1, 3, 4, 2).contiguous())
