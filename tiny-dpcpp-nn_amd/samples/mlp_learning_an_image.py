#!/usr/bin/env python3
"""Learns a 2-D image with a hash-grid encoding and a fused MLP, through the `tiny_dpcpp_nn` package on an MI355X.

Counterpart of samples/mlp_learning_an_image_pytorch.py of the reference (same model: 2-D HashGrid with 16 levels of 2
features, log2 hashmap size 15 by default, feeding a 64-wide network with 2 hidden layers; Adam, lr 1e-2; relative L2 loss;
batches of uniformly random pixel positions). By default the target is a procedural image (smooth colour fields with a few
sharp discs), evaluated analytically at the sampled positions, so that the sample runs without any file; `--image FILE`
learns a picture instead (anything Pillow opens, e.g. the reference's samples/data/images/albert.jpg), looked up with
bilinear filtering as the reference's sample does (:58-91 there). `--ppm out.ppm` writes the learned image.

    python tiny-dpcpp-nn_amd/samples/mlp_learning_an_image.py --n_steps 1000
    python tiny-dpcpp-nn_amd/samples/mlp_learning_an_image.py --image albert.jpg --ppm learned.ppm
"""
import argparse
import os
import sys
import time

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import tiny_dpcpp_nn as tnn  # noqa: E402

DTYPE = torch.bfloat16


def target_image(xy):
    """RGB in [0, 1] at positions xy in [0, 1]^2."""
    x, y = xy[:, 0], xy[:, 1]
    r = 0.5 + 0.5 * torch.sin(9.0 * x + 3.0 * y)
    g = 0.5 + 0.5 * torch.cos(7.0 * y) * torch.sin(5.0 * x * y + 1.0)
    b = x * (1 - y) + 0.3 * torch.sin(20.0 * (x - 0.5) ** 2 + 20.0 * (y - 0.5) ** 2)
    rgb = torch.stack([r, g, b.clamp(0, 1)], dim=1)
    for cx, cy, rad in ((0.3, 0.3, 0.08), (0.7, 0.6, 0.12), (0.5, 0.85, 0.05)):
        inside = ((x - cx) ** 2 + (y - cy) ** 2 < rad * rad).unsqueeze(1)
        rgb = torch.where(inside, 1.0 - rgb, rgb)
    return rgb


class PictureTarget:
    """A picture as a function on [0, 1]^2: the value at (x, y) blends the four pixels around (x * width, y * height), pixel
    (i, j) sitting at the integer position (i, j) and the last row and column repeated beyond the edge."""

    def __init__(self, filename, device):
        from PIL import Image  # only needed for --image

        rgb = Image.open(filename).convert("RGB")
        self.width, self.height = rgb.size
        pixels = torch.frombuffer(bytearray(rgb.tobytes()), dtype=torch.uint8).reshape(self.height * self.width, 3)
        self.pixels = (pixels.float() / 255.0).to(device)

    def __call__(self, xy):
        px = xy[:, 0] * self.width
        py = xy[:, 1] * self.height
        ix = px.floor().clamp(0, self.width - 1)
        iy = py.floor().clamp(0, self.height - 1)
        fx, fy = (px - ix).unsqueeze(1), (py - iy).unsqueeze(1)
        ix, iy = ix.long(), iy.long()
        jx, jy = (ix + 1).clamp(max=self.width - 1), (iy + 1).clamp(max=self.height - 1)
        top = torch.lerp(self.pixels[iy * self.width + ix], self.pixels[iy * self.width + jx], fx)
        bottom = torch.lerp(self.pixels[jy * self.width + ix], self.pixels[jy * self.width + jx], fx)
        return torch.lerp(top, bottom, fy)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--image", default=None, help="learn this picture instead of the procedural image")
    ap.add_argument("--n_steps", type=int, default=1000)
    ap.add_argument("--batch_size", type=int, default=2 ** 16)
    ap.add_argument("--log2_hashmap_size", type=int, default=15)
    ap.add_argument("--ppm", default=None, help="write the learned 512 x 512 image here")
    ap.add_argument("--seed", type=int, default=None, help="the same batches and the same initial weights in every run")
    args = ap.parse_args()
    if args.seed is not None:
        torch.manual_seed(args.seed)
        tnn.manual_seed(args.seed)

    device = "cuda"
    target = PictureTarget(args.image, device) if args.image else target_image
    encoding_config = {"otype": "HashGrid", "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": args.log2_hashmap_size,
                       "base_resolution": 16, "per_level_scale": 1.5}
    network_config = {"otype": "FullyFusedMLP", "activation": "ReLU", "output_activation": "None", "n_neurons": 64, "n_hidden_layers": 2}
    model = tnn.NetworkWithInputEncoding(2, 3, network_config, encoding_config, device=device, dtype=DTYPE, use_bias=False)
    optimizer = torch.optim.Adam(model.parameters(), lr=1e-2)

    interval, prev = 10, time.perf_counter()
    for i in range(args.n_steps):
        batch = torch.rand([args.batch_size, 2], device=device)
        targets = target(batch)
        output = model(batch).float()
        relative_l2_error = (output - targets) ** 2 / (output.detach() ** 2 + 0.01)
        loss = relative_l2_error.mean()
        optimizer.zero_grad()
        loss.backward()
        optimizer.step()
        if i % interval == 0 or i + 1 == args.n_steps:
            loss_val = loss.item()
            now = time.perf_counter()
            print(f"Step#{i}: loss={loss_val:.6f} time={int((now - prev) * 1e6)}[us]")
            prev = time.perf_counter()
            if i > 0 and interval < 1000:
                interval *= 10

    res = 512
    xs = (torch.arange(res, device=device) + 0.5) / res
    yv, xv = torch.meshgrid(xs, xs, indexing="ij")
    xy = torch.stack((xv.flatten(), yv.flatten()), dim=1)
    model.eval()
    with torch.no_grad():
        img = model(xy).float().clamp(0, 1)
    mse = float(((img - target(xy)) ** 2).mean())
    print(f"mean squared error of the learned {res} x {res} image: {mse:.6f}")
    if args.ppm:
        data = (img.reshape(res, res, 3) * 255).round().to(torch.uint8).cpu().numpy()
        with open(args.ppm, "wb") as f:
            f.write(f"P6 {res} {res} 255\n".encode())
            f.write(data.tobytes())
        print(f"wrote {args.ppm}")
    return mse


if __name__ == "__main__":
    main()
