"""Generates and compiles (hiprtc, gfx950) the kernels of the benchmark configurations into the on-disk
kernel cache, so that a GPU run starts without JIT latency. Needs no GPU."""
import time

from helium_amd import configs
from helium_amd.kernels import TileKernel
from helium_amd.permute import PermuteDims


def prebuild_kernels(verbose=True):
    t0 = time.time()
    n = 0
    for shape, perm in list(configs.PERMUTES.values()) + [((8192, 8192), (0, 1))]:
        PermuteDims(shape, "bf16", perm=perm)
        n += 1
    g, _, _ = configs.c3_chain(make_inputs=False)
    TileKernel.auxiliary(g)
    for mainloop, full in ((False, False), (True, True)):
        g, _ = configs.c4_graph(4096, mainloop=mainloop, full_size_outputs=full)
        TileKernel.fused(g)
        n += 1
    for g in (configs.c5a_graph(4096)[0], configs.c1_graph()[0]):
        TileKernel.fused(g)
        n += 1
    # the plans the benchmark runs through execute_graph
    from helium_amd import ir
    from helium_amd.backend import Plan
    from . import frontend

    Plan(configs.c1_ir_graph()[0]).precompile()
    g = ir.OpGraph()
    rec = frontend.Recorder(g)
    x = g.new_input([64, 56, 56, 256], "bf16")
    y, new_mean, new_var = frontend.batch_norm_train(rec, x, *[g.new_input([256], "f32") for _ in range(4)])
    for v in (y, new_mean, new_var):
        g.new_output(v)
    Plan(g).precompile()
    n += 2
    # one residual-block convolution and its two gradients, and the optimizer step of the largest filter
    conv = {"in_channels": 64, "out_channels": 64, "kernel_size": [3, 3]}
    for which in ("forward", "data", "filter"):
        g = ir.OpGraph()
        a = g.new_input([64, 56, 56, 64], "bf16")
        if which == "forward":
            out = g.conv(a, g.new_input([64, 3, 3, 64], "bf16"), conv)
        elif which == "data":
            out = g.conv_backward_data(a, g.new_input([64, 3, 3, 64], "bf16"), conv, [56, 56])
        else:
            out = g.conv_backward_filter(a, g.new_input([64, 56, 56, 64], "bf16"), conv)
        g.new_output(out)
        Plan(g).precompile()
        n += 1
    g = ir.OpGraph()
    rec = frontend.Recorder(g)
    out = g.conv(g.new_input([64, 56, 56, 64], "bf16"), g.new_input([64, 3, 3, 64], "bf16"), conv)
    g.new_output(out)
    for v in frontend.batch_norm_train(rec, out, *[g.new_input([64], "f32") for _ in range(4)]):
        g.new_output(v)
    Plan(g).precompile()
    n += 1
    g = ir.OpGraph()
    rec = frontend.Recorder(g)
    block = [[g.new_input([64], "f32") for _ in range(4)], g.new_input([64, 3, 3, 64], "bf16"), g.new_input([64], "bf16")]
    block += [[g.new_input([64], "f32") for _ in range(4)], g.new_input([64, 3, 3, 64], "bf16"), g.new_input([64], "bf16")]
    out, stats = frontend.basic_block_forward(rec, g.new_input([64, 56, 56, 64], "bf16"), *block)
    for v in [out] + stats:
        g.new_output(v)
    Plan(g).precompile()
    n += 1
    g = ir.OpGraph()
    rec = frontend.Recorder(g)
    shape = [512, 3, 3, 512]
    new_w, new_avg = frontend.sgd_momentum_step(rec, g.new_input(shape, "bf16"), g.new_input(shape, "bf16"), g.new_input(shape, "f32"))
    g.new_output(new_w)
    g.new_output(new_avg)
    Plan(g).precompile()
    n += 1
    # C5a and C4m the way the fusion search plans them
    from helium_amd import fusion_search as fs

    g, outs = configs.c4_graph(4096, mainloop=True, full_size_outputs=True)
    for node in ("loss", "db8", "db6"):
        g.consumer(outs[node], "f32")
    for g in (g, configs.c5a_graph(4096)[0]):
        fs.FusionPlan(g, fs.MIN_MI355X_COST).precompile()
        n += 1
    # the whole training step at the benchmark's two sizes and at the size the parity tests run it
    from . import resnet

    for kwargs in (dict(batch=128, image_size=224), dict(batch=64, image_size=256),
                   dict(batch=8, image_size=64, width=8, num_classes=16, dtype="f32"),
                   dict(batch=8, image_size=64, width=8, num_classes=16, dtype="bf16")):
        g = resnet.record_training_step(**kwargs)["graph"].g
        g.optimize()
        Plan(g).precompile()
        n += 1
    if verbose:
        print(f"prebuilt {n + 1} kernels in {time.time() - t0:.1f}s")
    return n + 1


if __name__ == "__main__":
    prebuild_kernels()
