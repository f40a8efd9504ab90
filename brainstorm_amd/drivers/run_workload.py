"""Runs training steps of one network workload on HipHandler: the program to put under a profiler.

    python3 -m brainstorm_amd.drivers.run_workload mlp|lstm|highway|cnn [steps] [fused] [recorded] [window_off] [im2col]

``fused`` is passed to the workload's builder: "0" for the reference layers' primitive call sequences
(what an unchanged caller issues), "1" for a handler-aware caller that asks for the fused entry points;
for the LSTM "packed" (stacked recurrent product), "thin" (packed, backward product through the
thin-operand kernel) or "sequence" (packed, forward recurrence in one launch). With "recorded" the step
is recorded after one ordinary step and replayed. With "window_off" the handler's fusing window is
switched off, so that primitive calls are launched one by one. With "im2col" convolutions with thin filters
take the col matrix and the matrix-product library like all others. One step = forward + backward + momentum
update.
"""
import sys

from brainstorm_amd import HipHandler
from brainstorm_amd.drivers import configs
from brainstorm_amd.drivers.net import MomentumStepper


def main(argv):
    name = argv[1]
    steps = int(argv[2]) if len(argv) > 2 else 3
    fused = argv[3] if len(argv) > 3 else ""
    kw = {}
    recorded = "recorded" in argv[4:]
    if fused and fused != "0":
        kw["fused"] = fused if fused in ("packed", "thin", "sequence") else True
    handler = HipHandler(seed=0, fusing="window_off" not in argv[4:])
    handler.thin_convolutions = "im2col" not in argv[4:]
    net, data = getattr(configs, "build_" + name)(handler, **kw)
    net.provide_external_data(data)
    stepper = MomentumStepper(0.1, 0.9, fused=bool(kw.get("fused")))
    stepper.start(net)
    if recorded:
        stepper.run()
    for _ in range(steps):
        if recorded:
            stepper.run_recorded()
        else:
            stepper.run()
    handler.synchronize()
    print("%s: %d steps done" % (name, steps))


if __name__ == "__main__":
    main(sys.argv)
