"""Small helpers shared by the modules (same names and meaning as the reference's
sparseconvnet/utils.py:11-26)."""
import glob
import os

import torch


def toLongTensor(dimension, x):
    """A CPU LongTensor of `dimension` sizes from an int, a list/tuple or a LongTensor."""
    if isinstance(x, torch.Tensor):
        if x.dtype != torch.int64 or x.is_cuda:
            x = x.detach().cpu().long()
        assert x.numel() == dimension
        return x
    if isinstance(x, (list, tuple)):
        assert len(x) == dimension
        return torch.tensor([int(v) for v in x], dtype=torch.int64)
    return torch.full((dimension,), int(x), dtype=torch.int64)


def optionalTensor(module, name):
    """module.<name> if it exists, else an empty tensor (how the reference passes 'no bias')."""
    return getattr(module, name) if hasattr(module, name) else torch.Tensor()


def optionalTensorReturn(a):
    return a if a.numel() else None


def prepare_BLInput(batch):
    """utils.py:127-136: pads a list of (locations [n_i, d], features [n_i, planes]) samples
    to one [batch, max n_i, d] location tensor (filled up with -1 = empty) and one
    [batch, max n_i, planes] feature tensor (filled up with zeros) for BLInputLayer."""
    with torch.no_grad():
        longest = max(loc.size(0) for loc, _ in batch)
        loc0, feat0 = batch[0]
        locations = torch.full((len(batch), longest, loc0.size(1)), -1, dtype=torch.int64)
        features = torch.zeros(len(batch), longest, feat0.size(1))
        for i, (loc, feat) in enumerate(batch):
            locations[i, :loc.size(0)] = loc
            features[i, :feat.size(0)] = feat
    return [locations, features]


def is_power2(num):
    """utils.py:157-158."""
    return num != 0 and ((num & (num - 1)) == 0)


def checkpoint_restore(model, exp_name, name2, use_cuda=True, epoch=0):
    """utils.py:138-155: loads `<exp_name>-<epoch, 9 digits>-<name2>.pth` (the newest one when
    epoch is 0) into the model and returns the epoch to continue with; 1 when there is none.
    The state dict is read with weights_only=True: parameter and buffer tensors only."""
    if use_cuda:
        model.cpu()
    if epoch > 0:
        f = exp_name + '-%09d-' % epoch + name2 + '.pth'
        assert os.path.isfile(f)
        print('Restore from ' + f)
        model.load_state_dict(torch.load(f, weights_only=True))
    else:
        found = sorted(glob.glob(exp_name + '-*-' + name2 + '.pth'))
        if len(found) > 0:
            f = found[-1]
            print('Restore from ' + f)
            model.load_state_dict(torch.load(f, weights_only=True))
            epoch = int(f[len(exp_name) + 1:-len(name2) - 5])
    if use_cuda:
        model.cuda()
    return epoch + 1


def checkpoint_save(model, exp_name, name2, epoch, use_cuda=True):
    """utils.py:166-177: saves the state dict and removes the previous epoch's file unless its
    number is a power of two."""
    f = exp_name + '-%09d-' % epoch + name2 + '.pth'
    model.cpu()
    torch.save(model.state_dict(), f)
    if use_cuda:
        model.cuda()
    epoch = epoch - 1
    f = exp_name + '-%09d-' % epoch + name2 + '.pth'
    if os.path.isfile(f) and not is_power2(epoch):
        os.remove(f)
