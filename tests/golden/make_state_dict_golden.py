"""Writes unet_state_dict.pth / unet_state_dict_io.npz: a small residual U-Net built by the
REFERENCE's own Python modules (sparseconvnet/networkArchitectures.py, sequential.py, ...), its
state dict as those modules name and shape it, a seeded input and the output the reference's CPU
path computes for it in eval mode.  A reference-trained checkpoint is such a state dict, so a
model of this repository that loads the file with strict key matching and reproduces the output
is compatible with one (sparseconvnet/utils.py:138-177 saves and restores exactly this).

Only this script touches the reference, and only in the container that holds its tree: it loads
the reference's CPU extension (sparseconvnet/SCN/pybind.cpp + sparseconvnet_cpu.cpp compiled where
they lie by oracle/Makefile, target _ref/SCN.so) and then imports the reference's Python package
from REF_ROOT.  The files it writes are data (tensors and arrays).  Run from the repository root:
    make -C oracle _ref/SCN.so && python tests/golden/make_state_dict_golden.py
"""
import importlib.util
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
HERE = os.path.dirname(os.path.abspath(__file__))
REF_ROOT = os.environ.get("REF_ROOT", "/root/reference")
sys.path.insert(0, ROOT)


def reference_package():
    so = os.path.join(ROOT, "oracle", "_ref", "SCN.so")
    spec = importlib.util.spec_from_file_location("sparseconvnet.SCN", so)
    ext = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ext)
    sys.modules["sparseconvnet.SCN"] = ext
    sys.path.insert(0, REF_ROOT)
    import sparseconvnet
    sparseconvnet.SCN = ext
    return sparseconvnet


def build(scn, m=8):
    """The same constructor calls on either package."""
    return scn.Sequential().add(scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
        scn.UNet(3, 1, [m, 2 * m, 3 * m], True)).add(scn.BatchNormReLU(m)).add(scn.OutputLayer(3))


def main():
    from sparseconvnet_amd import synthetic
    scn = reference_package()
    torch.manual_seed(77)
    model = build(scn)
    g = torch.Generator().manual_seed(78)
    with torch.no_grad():  # statistics and affine terms away from their initial 0 / 1
        for mod in model.modules():
            if hasattr(mod, "running_mean"):
                mod.running_mean.copy_(torch.randn(mod.running_mean.shape, generator=g) * 0.3)
                mod.running_var.copy_(torch.rand(mod.running_var.shape, generator=g) + 0.5)
                mod.weight.copy_(torch.rand(mod.weight.shape, generator=g) + 0.5)
                mod.bias.copy_(torch.randn(mod.bias.shape, generator=g) * 0.2)
    model.eval()
    coords = synthetic.room_scene(seed=7700, target=2500, spatial=32, n_boxes=5, duplicate_fraction=0.25)
    feats = np.random.default_rng(79).uniform(-1, 1, size=(len(coords), 3)).astype(np.float32)
    with torch.no_grad():
        x = scn.InputLayer(3, 32, mode=4)([torch.as_tensor(coords), torch.as_tensor(feats)])
        y = model(x)
    state = {k: v.detach().clone() for k, v in model.state_dict().items()}
    torch.save(state, os.path.join(HERE, "unet_state_dict.pth"))
    np.savez_compressed(os.path.join(HERE, "unet_state_dict_io.npz"), coords=coords, feats=feats, out=y.numpy())
    print("wrote %d tensors, %d points -> output %s" % (len(state), len(coords), tuple(y.shape)))
    for k, v in state.items():
        print("  %-40s %s" % (k, tuple(v.shape)))


if __name__ == "__main__":
    main()
