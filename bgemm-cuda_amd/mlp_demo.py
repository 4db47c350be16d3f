"""MLP classifier demo on the binary layers: train, evaluate, export the binary layers' weights as
bit-packed files and run inference from them.

Follows the reference's demo (tests/python/test_model_demo.py:107-151 model, :29-74 loops, :153-236
driver): a 512-128-128-128-1 MLP whose two middle layers are the selectable binary Linear, a float first
layer, batch norm + dropout + ReLU after every layer, a float head, BCE-with-logits loss, Adam with a
smaller learning rate for the layers' scale and zero-point parameters.  The reference trains on a
pre-binarised intrusion-detection table it loads from a file that is not part of its repository; here
the samples are synthetic with the same shape and value set ({-0.5, +0.5}^512, one 0/1 label) and a
label rule a small network can learn, so the demo runs anywhere and its result can be asserted.

    python mlp_demo.py bgemm_elastic --epochs 3 --export /tmp/mlp_packed
"""
import argparse
import os
import random
import time

import numpy as np
import torch
import torch.nn as nn
from torch.utils.data import DataLoader, TensorDataset

import lowbit_kernel
from bgemm_linear import (BGEMMLinear, BGEMMLinear_bireal, BGEMMLinear_elastic_signed, BNNLinear,
                          NNLinear_elastic_signed)

LINEARS = {                      # same model names as the reference's command line (test_model_demo.py:157-173)
    'bgemm_elastic': BGEMMLinear_elastic_signed,
    'nn_elastic': NNLinear_elastic_signed,
    'bgemm_bireal': BGEMMLinear_bireal,
    'bgemm': BGEMMLinear,
    'bnn_fp16': BNNLinear,
    'fp16': nn.Linear,
}
SCALE_PARAMS = ('sw', 'sa', 'zpw', 'zpa')


def seed_all(seed=1029):
    """Same seed for every generator the demo draws from (the reference's default, test_model_demo.py:19-27)."""
    os.environ['PYTHONHASHSEED'] = str(seed)
    for set_seed in (random.seed, np.random.seed, torch.manual_seed):
        set_seed(seed)                    # torch.manual_seed also seeds every GPU's generator


def synthetic_dataset(samples, features=512, seed=0):
    """`samples` (rounded down to a multiple of 32, as the reference does) rows of +-0.5 with a 0/1 label:
    the label says whether more of the first 64 features are +0.5 than of the next 64."""
    g = torch.Generator().manual_seed(seed)
    samples = samples // 32 * 32
    x = torch.randint(0, 2, (samples, features), generator=g).to(torch.float16) - 0.5
    y = (x[:, :64].float().sum(1) > x[:, 64:128].float().sum(1)).to(torch.float16)
    return TensorDataset(x, y)


class FC_half2float(nn.Linear):
    """Float head whatever the dtype of the features (test_model_demo.py:102-112)."""

    def __init__(self, in_channels, out_channels, bias=False):
        super().__init__(in_channels, out_channels, bias)

    def forward(self, x):
        out = nn.functional.linear(x.float(), self.weight.float())
        return out if self.bias is None else out + self.bias.view(1, -1)


class MLP(nn.Module):
    """Three stages of (linear, batch norm, dropout, ReLU) and a float head.  Only the first stage's linear is
    always full precision; `Linear` picks the kind of the other two.  Attribute names are the reference's
    (lin1..3, bn1..3, fc), so its state dicts load."""

    def __init__(self, Linear=BGEMMLinear, dtype=torch.half, bias=True,
                 input_size=512, hidden1=128, hidden2=128, hidden3=128, num_classes=1):
        super().__init__()
        widths = (input_size, hidden1, hidden2, hidden3)
        for stage, kind in enumerate((nn.Linear, Linear, Linear), start=1):
            self.add_module("lin%d" % stage, kind(widths[stage - 1], widths[stage], bias=bias))
            self.add_module("bn%d" % stage, nn.BatchNorm1d(widths[stage]))
        self.fc = FC_half2float(hidden3, num_classes, bias=True)
        self.act = nn.Sequential(nn.Dropout(0.5), nn.ReLU())

    def forward(self, x):
        for stage in (1, 2, 3):
            x = self.act(getattr(self, "bn%d" % stage)(getattr(self, "lin%d" % stage)(x)))
        return self.fc(x)


def train(model, loader, optimizer, criterion, device, dtype=torch.float):
    model.train()
    losses = []
    for inputs, target in loader:
        inputs, target = inputs.to(device), target.to(device)
        optimizer.zero_grad()
        loss = criterion(model(inputs.to(dtype)), target.unsqueeze(1).float())
        loss.backward()
        optimizer.step()
        losses.append(loss.detach())
    return torch.stack(losses).cpu().tolist()


def test(model, loader, device, dtype=torch.float):
    """Accuracy of sigmoid(output) > 0.5 against the 0/1 labels."""
    model.eval()
    right = total = 0
    with torch.no_grad():
        for inputs, target in loader:
            inputs, target = inputs.to(device), target.to(device)
            pred = torch.sigmoid(model(inputs.to(dtype))).reshape(-1) > 0.5
            right += int((pred == (target > 0.5)).sum())
            total += target.numel()
    return right / max(total, 1)


def make_optimizer(model, lr=1e-3, scale_lr=1e-4):
    named = list(model.named_parameters())
    is_scale = lambda n: any(s in n for s in SCALE_PARAMS)
    groups = [{'params': [p for n, p in named if is_scale(n)], 'lr': scale_lr},
              {'params': [p for n, p in named if not is_scale(n)]}]
    return torch.optim.Adam(groups, lr=lr, betas=(0.9, 0.999))


def export_packed(model, directory):
    """Write every sign-binarised layer's centred weight as a bit-packed file (1 bit per weight, the layout
    the kernels stream) and return the paths.  Layers that ternarise or keep float weights are skipped."""
    os.makedirs(directory, exist_ok=True)
    paths = {}
    for name, mod in model.named_modules():
        if isinstance(mod, BGEMMLinear) and mod.initialized:
            paths[name] = os.path.join(directory, name.replace('.', '_') + ".bgemmpk")
            lowbit_kernel.save_packed(paths[name], mod._packed_weight())
    return paths


def import_packed(model, paths, device):
    """Install packed weight files as the layers' cached packed operand: inference then never touches
    the float weights."""
    for name, mod in model.named_modules():
        if name in paths:
            mod.use_packed_weight(lowbit_kernel.load_packed(paths[name], device))


def run(model_name='bgemm_elastic', epochs=3, train_samples=8192, test_samples=2048, batch_size=256,
        device=None, dtype=torch.float, seed=0, export=None, log=print):
    device = torch.device(device or ("cuda" if torch.cuda.is_available() else "cpu"))
    if device.type != "cuda" and model_name.startswith("bgemm"):
        raise RuntimeError("the bgemm layers need the GPU library; choose bnn_fp16, nn_elastic or fp16 on a CPU")
    seed_all(seed)
    mlp = MLP(Linear=LINEARS[model_name], dtype=dtype, bias=True).to(device)
    train_loader = DataLoader(synthetic_dataset(train_samples, seed=seed + 1), batch_size=batch_size, shuffle=True)
    test_loader = DataLoader(synthetic_dataset(test_samples, seed=seed + 2), batch_size=batch_size, shuffle=False)
    criterion = nn.BCEWithLogitsLoss().to(device)
    optimizer = make_optimizer(mlp)
    history = []
    t0 = time.time()
    for epoch in range(epochs):
        losses = train(mlp, train_loader, optimizer, criterion, device, dtype)
        acc = test(mlp, test_loader, device, dtype)
        history.append((float(np.mean(losses)), acc))
        log("epoch %d  training loss = %f  test accuracy = %f" % (epoch, history[-1][0], acc))
    log("total training time: %.3f s" % (time.time() - t0))
    result = {"model": model_name, "history": history, "accuracy": history[-1][1] if history else None, "mlp": mlp,
              "test_loader": test_loader}
    if export:
        paths = export_packed(mlp, export)
        import_packed(mlp, paths, device)
        result["packed_files"] = paths
        result["accuracy_from_packed"] = test(mlp, test_loader, device, dtype)
        log("exported %d packed layers to %s; accuracy from the packed files = %f"
            % (len(paths), export, result["accuracy_from_packed"]))
    return result


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("model", nargs="?", default="bgemm_elastic", choices=sorted(LINEARS))
    ap.add_argument("--epochs", type=int, default=20)
    ap.add_argument("--train-samples", type=int, default=65536)
    ap.add_argument("--test-samples", type=int, default=8192)
    ap.add_argument("--batch-size", type=int, default=256)
    ap.add_argument("--export", default=None, help="directory for the bit-packed weights of the binary layers")
    a = ap.parse_args(argv)
    run(a.model, a.epochs, a.train_samples, a.test_samples, a.batch_size, export=a.export)


if __name__ == "__main__":
    main()
