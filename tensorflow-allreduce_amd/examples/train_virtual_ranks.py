#!/usr/bin/env python3
"""Data-parallel training over virtual ranks on one MI355X.

The torch counterpart of the example in the reference's package docstring
(tensorflow/contrib/mpi_collectives/__init__.py:83-109): every rank holds a
replica of the model, computes gradients on its own batch, and a
DistributedOptimizer averages the gradients with ring allreduces before the
update. Here the ranks are virtual: one process, one GPU.

    python tensorflow-allreduce_amd/examples/train_virtual_ranks.py [--ranks 4] [--steps 20] [--fusion]
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import torch  # noqa: E402

import mpi_collectives as mpi  # noqa: E402


def make_model():
    return torch.nn.Sequential(torch.nn.Linear(64, 128), torch.nn.ReLU(), torch.nn.Linear(128, 10)).cuda()


def batch_for_rank(rank, step, n=32):
    """On different ranks, feed different input data."""
    gen = torch.Generator().manual_seed(1000 * step + rank)
    x = torch.randn(n, 64, generator=gen)
    y = (x[:, :10].argmax(dim=1)).long()
    return x.cuda(), y.cuda()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ranks", type=int, default=4)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--fusion", action="store_true",
                    help="let the coordinator fuse each step's gradient allreduces into one ring")
    args = ap.parse_args()

    torch.manual_seed(0)
    reference = make_model()
    models, optimizers = [], []
    for _ in range(args.ranks):
        m = make_model()
        m.load_state_dict(reference.state_dict())           # every rank starts from the same weights
        models.append(m)
        # MPI allreduce the gradients before applying them
        optimizers.append(mpi.DistributedOptimizer(torch.optim.SGD(m.parameters(), lr=0.1)))
    loss_fn = torch.nn.CrossEntropyLoss()

    with mpi.Session(size=args.ranks, fusion_threshold=(8 << 20) if args.fusion else 0) as session:
        for step in range(args.steps):
            grads, losses = [], []
            for r in range(args.ranks):                     # what each MPI process would do
                with session.as_rank(r):
                    optimizers[r].zero_grad()
                    x, y = batch_for_rank(mpi.rank(), step)
                    loss = loss_fn(models[r](x), y)
                    grads.append(optimizers[r].compute_gradients(loss))
                    # average loss for printing: an allreduce of a scalar tensor
                    losses.append(mpi.allreduce(loss.detach().reshape(1)))
            avg_loss = session.run(losses)[0].item()        # every collective of this step runs here
            for r in range(args.ranks):
                with session.as_rank(r):
                    optimizers[r].apply_gradients(grads[r])
            if step % 5 == 0 or step == args.steps - 1:
                print("step %3d  average loss %.4f" % (step, avg_loss))
    # the replicas saw the same averaged gradients, so they stayed identical
    for m in models[1:]:
        for p, q in zip(models[0].parameters(), m.parameters()):
            assert torch.equal(p, q)
    print("all %d replicas hold identical weights" % args.ranks)
    return avg_loss


if __name__ == "__main__":
    main()
