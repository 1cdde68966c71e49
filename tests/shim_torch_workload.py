"""A PyTorch-ROCm program that knows nothing of XSched: a few training steps of a small network
on a side stream, with a second stream and events next to it. tests/test_gpu_shim.py runs it
with and without the interception shim preloaded and compares what it prints."""
import hashlib
import sys

import torch


def digest(t):
    return hashlib.sha256(t.detach().float().cpu().numpy().tobytes()).hexdigest()[:16]


def timed(steps=200, rounds=5):
    """`--time`: the same network trained for `rounds` x `steps` steps on a side stream, the
    median round in microseconds per step (bench.py runs it natively and under the shim)."""
    import time
    torch.manual_seed(0)
    dev = torch.device("cuda")
    work = torch.cuda.Stream()
    with torch.cuda.stream(work):
        model = torch.nn.Sequential(torch.nn.Linear(256, 512), torch.nn.ReLU(),
                                    torch.nn.Linear(512, 512), torch.nn.Tanh(),
                                    torch.nn.Linear(512, 10)).to(dev)
        opt = torch.optim.SGD(model.parameters(), lr=0.05, momentum=0.9)
        x = torch.randn(1024, 256, device=dev)
        y = torch.randint(0, 10, (1024,), device=dev)

        def train(n):
            for _ in range(n):
                opt.zero_grad()
                loss = torch.nn.functional.cross_entropy(model(x), y)
                loss.backward()
                opt.step()
            return loss

        train(50)
        work.synchronize()
        per_step = []
        for _ in range(rounds):
            t0 = time.perf_counter()
            loss = train(steps)
            work.synchronize()
            per_step.append((time.perf_counter() - t0) * 1e6 / steps)
    print("timed steps=%d rounds=%d us_per_step=%.1f loss=%.6f" % (steps, rounds, sorted(per_step)[rounds // 2], loss.item()))


def main():
    if len(sys.argv) > 1 and sys.argv[1] == "--time":
        return timed()
    torch.manual_seed(0)
    dev = torch.device("cuda")
    work, side = torch.cuda.Stream(), torch.cuda.Stream()
    done = torch.cuda.Event()
    with torch.cuda.stream(work):
        model = torch.nn.Sequential(torch.nn.Linear(256, 512), torch.nn.ReLU(),
                                    torch.nn.Linear(512, 512), torch.nn.Tanh(),
                                    torch.nn.Linear(512, 10)).to(dev)
        opt = torch.optim.SGD(model.parameters(), lr=0.05, momentum=0.9)
        x = torch.randn(1024, 256, device=dev)
        y = torch.randint(0, 10, (1024,), device=dev)
        losses = []
        for _ in range(40):
            opt.zero_grad()
            loss = torch.nn.functional.cross_entropy(model(x), y)
            loss.backward()
            opt.step()
            losses.append(loss.detach())
        done.record(work)
    with torch.cuda.stream(side):
        side.wait_event(done)                      # the side stream reads what the work stream wrote
        norms = torch.stack([p.detach().norm() for p in model.parameters()])
        total = torch.stack(losses).sum()
    side.synchronize()
    host = torch.empty(6, pin_memory=True)
    with torch.cuda.stream(side):
        host.copy_(norms, non_blocking=True)       # device to pinned memory
    side.synchronize()
    print("losses", digest(torch.stack(losses)), "first %.6f last %.6f" % (losses[0].item(), losses[-1].item()))
    print("weights", " ".join(digest(p) for p in model.parameters()))
    print("norms", digest(host), "sum of losses", digest(total))
    assert losses[-1].item() < losses[0].item()
    print("done")


if __name__ == "__main__":
    sys.exit(main())
