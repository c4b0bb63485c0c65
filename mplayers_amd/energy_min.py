"""Energy minimisation with the message-passing layers: the reference's driver
(MPLayers/main.py:78-340) on this library, start to end on the GPU.

  terms      stereo data cost of an image pair (compute_terms.compute_terms_py) or a denoising
             unary from a CSV file (parse_unary_cost, main.py:24-40), or a synthetic random-dot
             stereo pair (no data set ships with the library)
  inference  MPModule (TRWP | ISGMR | SGM) in eval mode, saving the labelling of every iteration
  result     the energies of those labellings (the reference computes them off-line from the
             .mat file, tools/matlab/MRF/calEnergy.m) and, with --enable_saving_label, the .mat
             file with the reference's keys (main.py:326-336) plus `energy`

    python -m mplayers_amd.energy_min --synthetic 240 320 --mode TRWP --n_dir 8 --n_iter 20 \\
        --n_disp 32 --context TL --truncated 2 --p_weight 10
"""
import argparse
import csv
import os
import sys
import time

import numpy as np
import torch

from . import compute_terms
from .label_context import create_label_context
from .MP_module import MPModule


def parse_unary_cost(file_path):
  """CSV unary of the denoising problems: first line `height,width,n_disp`, then one line of
  n_disp costs per pixel in row-major order -> (height, width, n_disp, (H, W, L) fp32 tensor)."""
  with open(file_path, 'r') as f:
    rows = list(csv.reader(f, delimiter=','))
  height, width, n_disp = (int(v) for v in rows[0])
  if len(rows) - 1 != height * width:
    raise RuntimeError('%s: %d cost lines for %d pixels' % (file_path, len(rows) - 1, height * width))
  cost = np.array([[float(v) for v in row] for row in rows[1:]], dtype=np.float32)
  return height, width, n_disp, torch.from_numpy(cost.reshape(height, width, n_disp))


def synthetic_stereo_pair(height, width, n_disp, seed=2019, bands=3):
  """Random-dot stereogram: a textured left image and a right image in which rectangles of the
  scene are displaced by their disparity.  -> left, right (H, W, bands) uint8, disparity (H, W)."""
  rng = np.random.default_rng(seed)
  right = rng.integers(0, 256, size=(height, width + n_disp, bands), dtype=np.uint8)
  disparity = np.full((height, width), max(1, n_disp // 8), dtype=np.int64)
  for _ in range(6):
    h0, h1 = np.sort(rng.integers(0, height, size=2))
    w0, w1 = np.sort(rng.integers(0, width, size=2))
    disparity[h0:h1 + 1, w0:w1 + 1] = rng.integers(0, n_disp)
  cols = np.arange(width)[None, :] + n_disp - disparity       # left(x) = right(x - d)
  left = right[np.arange(height)[:, None], cols]
  return np.ascontiguousarray(left), np.ascontiguousarray(right[:, n_disp:]), disparity


def build_parser():
  parser = argparse.ArgumentParser(description='energy minimisation on a grid MRF')
  parser.add_argument('--data_dir', type=str, default='../datasets')
  parser.add_argument('--img_name', type=str, default='tsukuba')
  parser.add_argument('--mode', type=str, default='TRWP', choices=['TRWP', 'ISGMR', 'SGM'])
  parser.add_argument('--n_dir', type=int, default=4)
  parser.add_argument('--n_iter', type=int, default=50)
  parser.add_argument('--context', type=str, default='TL')
  parser.add_argument('--rho', type=float, default=None)
  parser.add_argument('--enable_min_a_dir', action='store_true', default=False)
  parser.add_argument('--enable_saving_label', action='store_true', default=False)
  parser.add_argument('--truncated', type=int, default=1)
  parser.add_argument('--n_disp', type=int, default=10)
  parser.add_argument('--p_weight', type=int, default=10)
  parser.add_argument('--left_img_path', type=str, default=None)
  parser.add_argument('--right_img_path', type=str, default=None)
  parser.add_argument('--save_dir', type=str, default='../experiments')
  parser.add_argument('--synthetic', type=int, nargs=2, metavar=('H', 'W'), default=None,
                      help='use a random-dot stereo pair of this size instead of image files')
  return parser


def _image_paths(args):
  """Where the reference looks for its data sets (main.py:131-150)."""
  if args.left_img_path is not None and args.right_img_path is not None:
    return args.left_img_path, args.right_img_path
  name, root = args.img_name, args.data_dir
  if name.startswith('000'):
    return (os.path.join(root, 'KITTI2015/image_2/%s.png' % name),
            os.path.join(root, 'KITTI2015/image_3/%s.png' % name))
  if name.split('_')[-1][-2:] in ('1l', '2l', '3l', '1s', '2s', '3s'):
    return (os.path.join(root, 'ETH3D/training/%s/im0.png' % name),
            os.path.join(root, 'ETH3D/training/%s/im1.png' % name))
  ext = 'pgm' if name == 'map' else 'ppm'
  return (os.path.join(root, 'Middlebury/%s/imL.%s' % (name, ext)),
          os.path.join(root, 'Middlebury/%s/imR.%s' % (name, ext)))


def build_terms(args):
  """-> unary (H, W, L) fp32 on the GPU, pairwise table (L, L) fp32 on the GPU (already scaled by
  p_weight), n_disp."""
  device = torch.device('cuda', torch.cuda.current_device())
  if args.synthetic is None and args.img_name in ('house', 'penguin'):
    path = '%s/Denoise/%s_unary.csv' % (args.data_dir, args.img_name)
    _, _, n_disp, cost = parse_unary_cost(path)
    # the denoising problems build their pairwise table with the label-context builder
    # (main.py:112-127): the term weight is applied there and the truncation acts on the
    # (squared) cost itself, a negative value meaning none
    ctx_args = argparse.Namespace(
        n_classes=n_disp, mpnet_smoothness_mode=args.context, mpnet_smoothness_train=None,
        mpnet_smoothness_trunct_loc=-1, mpnet_smoothness_trunct_value=args.truncated,
        mpnet_term_weight=args.p_weight, enable_cuda=False)
    table, _, _ = create_label_context(ctx_args, enable_seg=True, enable_symmetric=True)
    return cost.to(device), table.detach().to(device), n_disp
  if args.synthetic is not None:
    left, right, _ = synthetic_stereo_pair(args.synthetic[0], args.synthetic[1], args.n_disp)
  else:
    left, right = _image_paths(args)
    for path in (left, right):
      if not os.path.exists(path):
        raise RuntimeError('image %s does not exist' % path)
  param = compute_terms.MRFParams(left, right, args.context, args.n_disp, 0, 0, args.truncated)
  cost, _, table, _ = compute_terms.compute_terms_py(param)
  return cost, table * args.p_weight, args.n_disp


def minimise(args, unary, table, n_disp):
  """Runs the layer; -> labels (n_iter, H, W) uint8, energy (n_iter, 2) fp64 (unary, pairwise),
  cost_final (L, H, W), seconds."""
  n_dir, n_iter = args.n_dir, args.n_iter
  height, width = unary.shape[:2]
  module_args = argparse.Namespace(
      n_classes=n_disp, mpnet_n_dirs=n_dir, mpnet_max_iter=n_iter, mpnet_term_weight=args.p_weight,
      mpnet_smoothness_train=None, mpnet_mrf_mode=args.mode, rho=args.rho)
  module = MPModule(module_args, enable_create_label_context=False, enable_saving_label=True,
                    enable_min_a_dir=args.enable_min_a_dir)
  # one table per direction, as the reference driver passes it (main.py:177-178); the kernels read
  # the first one
  label_context = table.view(1, n_disp, n_disp).repeat(n_dir, 1, 1).contiguous()
  module.set_label_context(label_context, None, None)
  module.eval()
  volume = unary.permute(2, 0, 1).contiguous().view(1, 1, n_disp, height, width)
  torch.cuda.synchronize()
  start = time.time()
  with torch.no_grad():
    cost_final, _, label_all, _, _ = module(volume)
  torch.cuda.synchronize()
  seconds = time.time() - start
  labels = label_all.view(n_iter, 1, height, width)
  energy = compute_terms.mrf_energy(unary.view(1, height, width, n_disp).contiguous(),
                                    label_context, labels, None, n_dir)
  return labels.view(n_iter, height, width), energy, cost_final.view(n_disp, height, width), seconds


def result_path(args, rho):
  """File name of the reference's result (main.py:163-168)."""
  name = '%s_%s_iter_%d_%s_trunc_%d_dir_%d_rho_%s' % (args.img_name, args.mode, args.n_iter,
                                                      args.context, args.truncated, args.n_dir, rho)
  if args.enable_min_a_dir:
    name += '_minAdir'
  return os.path.join('%s/energy/%s' % (args.save_dir, args.img_name), name + '.mat')


def main(argv=None):
  args = build_parser().parse_args(argv)
  if args.n_disp > 256:
    raise RuntimeError('at most 256 labels')
  if not torch.cuda.is_available():
    raise RuntimeError('energy_min needs a GPU (there is no CPU path in this build)')
  if args.synthetic is not None and args.img_name == 'tsukuba':
    args.img_name = 'synthetic'
  if args.mode == 'SGM' and args.n_iter != 1:
    # SGM is one Jacobi iteration by definition; the reference moves this mode to its CPU path
    # because its GPU module insists on a single iteration (MP_module.py:205-206, main.py:239-241)
    print('SGM: running 1 iteration instead of %d' % args.n_iter)
    args.n_iter = 1
  # MPModule fixes rho per mode as the reference's does; the option only names the result file
  rho = args.rho if args.rho is not None else (0.5 if args.mode == 'TRWP' else 1)
  file_path = result_path(args, rho) if args.enable_saving_label else None
  if file_path is not None and os.path.exists(file_path):
    print('%s exist, exit.' % file_path)
    return None
  unary, table, n_disp = build_terms(args)
  labels, energy, cost_final, seconds = minimise(args, unary, table, n_disp)
  energy_host = energy.cpu().numpy()
  total = energy_host.sum(axis=1)
  print('%s, %d directions, %d iterations on %dx%dx%d: %.4f s' %
        (args.mode, args.n_dir, args.n_iter, unary.shape[0], unary.shape[1], n_disp, seconds))
  for it in sorted(set([0, args.n_iter // 2, args.n_iter - 1])):
    print('iteration %3d: energy %.6g (unary %.6g, pairwise %.6g)' %
          (it + 1, total[it], energy_host[it, 0], energy_host[it, 1]))
  if file_path is not None:
    import scipy.io as scio
    os.makedirs(os.path.dirname(file_path), exist_ok=True)
    scio.savemat(file_path, {
        'n_iter': args.n_iter, 'n_dir': args.n_dir, 'rho': rho, 'p_func': args.context,
        'n_disp': n_disp, 'p_weight': args.p_weight, 'trunct': args.truncated,
        'min_a_dir': int(args.enable_min_a_dir),
        'unary': unary.cpu().numpy(),
        'label_context': table.view(1, n_disp, n_disp).repeat(args.n_dir, 1, 1)
                              .permute(1, 2, 0).cpu().numpy(),
        'seg_all': labels.permute(1, 2, 0).cpu().numpy().astype(np.uint8),
        'energy': energy_host})
    print('saved %s' % file_path)
  return {'labels': labels, 'energy': energy, 'cost_final': cost_final, 'seconds': seconds,
          'file_path': file_path}


if __name__ == '__main__':
  main(sys.argv[1:])
