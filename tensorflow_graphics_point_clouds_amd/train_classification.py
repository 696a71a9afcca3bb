"""Training loop of the reference's classification script (modelnet40.py:400-560)
on this package's layers: RMSprop with a staircase exponential decay of the
learning rate, softmax cross-entropy, anisotropic scaling as augmentation.

No dataset ships with the package.  Without --files the script trains on a
seeded four-class set of geometric primitives; with --files it reads ASCII
clouds `x,y,z[,...]` whose class is the integer before the first '_' or '.' of
the file name modulo --classes.

    python -m tensorflow_graphics_point_clouds_amd.train_classification --epochs 3
"""
import argparse
import os
import time

import numpy as np
import torch

from . import io, models, synthetic


def batches(points, labels, batch_size, rng, augment):
    order = rng.permutation(len(points))
    for b in range(len(points) // batch_size):
        pick = order[b * batch_size:(b + 1) * batch_size]
        pts = points[pick].copy()
        if augment:                                        # modelnet40.py:437-440
            pts *= rng.uniform(0.9, 1.1, (len(pick), 1, 3)).astype(np.float32)
        yield pts, labels[pick]


def run_epoch(model, points, labels, batch_size, rng, optimizer=None, device="cuda"):
    training = optimizer is not None
    model.train(training)
    loss_sum = hits = seen = 0
    for pts, lab in batches(points, labels, batch_size, rng, augment=training):
        tp, tl = torch.as_tensor(pts, device=device), torch.as_tensor(lab, device=device)
        with torch.set_grad_enabled(training):
            logits = model(tp, training=training)
            loss = torch.nn.functional.cross_entropy(logits, tl)
        if training:
            optimizer.zero_grad(set_to_none=True)
            loss.backward()
            optimizer.step()
        loss_sum += float(loss.detach()) * len(lab)
        hits += int((logits.argmax(1) == tl).sum())
        seen += len(lab)
    return loss_sum / max(seen, 1), hits / max(seen, 1)


def load_files(paths, points_per_cloud, classes):
    pts, labels = [], []
    for path in paths:
        p, _ = io.load_points_from_file_to_numpy(path, max_num_points=points_per_cloud)
        if len(p) < points_per_cloud:
            raise ValueError(f"{path} holds fewer than {points_per_cloud} points")
        stem = os.path.basename(path).split("_")[0].split(".")[0]
        pts.append(p)
        labels.append(int(stem) % classes)
    return np.stack(pts), np.asarray(labels, dtype=np.int64)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--layer", default="MCConv", choices=["MCConv", "KPConv", "PointConv"])
    ap.add_argument("--epochs", type=int, default=3)
    ap.add_argument("--batch-size", type=int, default=16)
    ap.add_argument("--points", type=int, default=1024, help="points per cloud")
    ap.add_argument("--clouds", type=int, default=256, help="synthetic training clouds")
    ap.add_argument("--classes", type=int, default=4)
    ap.add_argument("--files", nargs="*", default=None)
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args(argv)

    if args.files:
        points, labels = load_files(args.files, args.points, args.classes)
        split = max(args.batch_size, int(0.8 * len(points)))
        train, test = (points[:split], labels[:split]), (points[split:], labels[split:])
    else:
        train = synthetic.labelled_primitives(args.clouds, args.points, args.seed)
        test = synthetic.labelled_primitives(max(args.clouds // 4, args.batch_size), args.points,
                                             args.seed + 1)
    rng = np.random.default_rng(args.seed)
    pool_radii = np.array([0.1, 0.2, 0.4])                 # the small set-up of modelnet40.py:547-548
    model = models.ClassificationNet([64, 128, 256, 128, args.classes], pool_radii,
                                     pool_radii * 2.0, layer_type=args.layer, dropout_rate=0.5,
                                     seed=args.seed)
    steps_per_epoch = max(len(train[0]) // args.batch_size, 1)
    optimizer = torch.optim.RMSprop(model.parameters(), lr=1e-3, alpha=0.9, eps=1e-7)
    schedule = torch.optim.lr_scheduler.StepLR(optimizer, step_size=20, gamma=0.7)
    for epoch in range(args.epochs):
        start = time.time()
        tr = run_epoch(model, *train, args.batch_size, rng, optimizer)
        te = run_epoch(model, *test, args.batch_size, rng) if len(test[0]) >= args.batch_size \
            else (float("nan"), float("nan"))
        schedule.step()
        print("epoch %03d  %.1fs  %d steps  train loss %.3f acc %.1f%%  test loss %.3f acc %.1f%%"
              % (epoch, time.time() - start, steps_per_epoch, tr[0], 100 * tr[1], te[0],
                 100 * te[1]), flush=True)
    return tr, te


if __name__ == "__main__":
    main()
