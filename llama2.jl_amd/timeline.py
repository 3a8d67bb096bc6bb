"""Where the time of one token goes inside the streaming decode kernel (launch path 3).

    python llama2.jl_amd/build.py --timeline          # builds llama2.jl_amd/libl2hip_tl.so (-DL2H_TIMELINE)
    python llama2.jl_amd/timeline.py [n_layers [plan]] # on the GPU; prints the table (plan: a name from synth.py, default PLAN_Q4_K_S)

In the profiling build thread 0 of every workgroup stamps the 100 MHz wall clock at the phase boundaries
of the first layers of a launch (after staging a phase's input, after the wait for the ring's pieces, at
the end of its own streaming loop, when the whole workgroup has finished it, after the epilogue).  The
script decodes a few tokens of a model with the benchmark's widths, reads the stamps of the last launch
and prints, per boundary, the minimum / median / maximum over the workgroups, the step from the previous
boundary (median), a one-line summary of a steady-state layer, the steps inside the attention of one layer
and the steps inside the staging function of one workgroup.  Numbers are microseconds since the first
workgroup started."""
import ctypes
import importlib.util
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
PHASES = ("qkv", "wo", "w13", "w2")
STAMPS = ("staged", "drained", "looped", "alldone", "fin")


def main():
    os.environ.setdefault("L2H_LIB", os.path.join(HERE, "libl2hip_tl.so"))
    spec = importlib.util.spec_from_file_location("llama2_jl_amd", os.path.join(HERE, "__init__.py"),
                                                  submodule_search_locations=[HERE])
    pkg = importlib.util.module_from_spec(spec)
    sys.modules["llama2_jl_amd"] = pkg
    spec.loader.exec_module(pkg)
    from llama2_jl_amd import _lib, synth
    n_layers = int(sys.argv[1]) if len(sys.argv) > 1 else 4
    plan = getattr(synth, sys.argv[2]) if len(sys.argv) > 2 else synth.PLAN_Q4_K_S  # e.g. PLAN_Q5_K_M: typed pieces
    cfg = pkg.ModelConfig(dim=4096, hidden_dim=14336, n_layers=n_layers, n_heads=32, n_kv_heads=8, vocab_size=128256,
                          seq_len=512, rope_freq_base=500000.0)
    lm = synth.synthetic_model(cfg, plan, seed=1)
    dev = lm.device(path=3)
    dev.generate_greedy(synth.seeded_prompt(1, 32, cfg.vocab_size), 8)
    lib = _lib.lib()
    if not hasattr(lib, "l2h_debug_timeline"):
        sys.exit("this library was built without -DL2H_TIMELINE: python llama2.jl_amd/build.py --timeline")
    lib.l2h_debug_timeline.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
    n_wg = dev.ctx.device_info()["n_cu"] if isinstance(dev.ctx.device_info(), dict) else 256
    buf = np.zeros(n_wg * 64 + 1024, np.int64)
    assert lib.l2h_debug_timeline(dev.handle, buf.ctypes.data_as(ctypes.c_void_p), n_wg) == 0
    tl = buf[:n_wg * 64].reshape(n_wg, 64)
    us = (tl - tl[:, 0].min()) * 0.01
    # the workgroups that run a head's attention have one more stamp per layer than the others
    stride = n_wg // cfg.n_heads
    att = np.array([(w // stride < cfg.n_heads) and (w % stride == (w // stride) % stride) for w in range(n_wg)])
    names = ["start"]
    for l in range(3):
        for ph in PHASES:
            if ph == "wo":
                names.append("att done l%d" % l)
            names += ["%s %s l%d" % (ph, st, l) for st in STAMPS]
    prev = None
    for i, nm in enumerate(names[:60]):
        col = us[~att, i]
        med = float(np.median(col))
        print("%-18s min %7.2f  med %7.2f  max %7.2f  step %5.2f | attention workgroups: med %7.2f"
              % (nm, col.min(), med, col.max(), med - prev if prev is not None else 0.0, float(np.median(us[att, i]))))
        prev = med
    med = np.median(us[~att], axis=0)
    per = len(PHASES) * len(STAMPS) + 1
    i0 = 1 + per  # layer 1: steady state
    if n_layers >= 3:
        d = np.diff(med[i0 - 1:i0 + per])
        print("layer 1: %.2f us = " % (med[i0 + per - 1] - med[i0 - 1]) +
              " ".join("%s:%.2f" % (names[i0 + k].rsplit(" ", 1)[0].replace(" ", "/"), d[k]) for k in range(per)))
    # inside the attention of layer 2 (short caches): five stamps per head, relative to the moment the head's
    # workgroup finished its q|k|v epilogue
    if n_layers >= 3:
        t0 = tl[:, 0].min()
        a_us = (buf[n_wg * 64:n_wg * 64 + cfg.n_heads * 16].reshape(cfg.n_heads, 16) - t0) * 0.01
        i_fin = names.index("qkv fin l2")
        wg_of = [h * stride + h % stride for h in range(cfg.n_heads)]
        rel = a_us[:, :5] - us[wg_of, i_fin][:, None]
        labels = ("entered", "q, k, v and the keys there", "scores and maximum", "softmax", "values summed")
        print("attention of layer 2, us after the workgroup's q|k|v epilogue (median over the heads): " +
              ", ".join("%s %.2f" % (lab, float(np.median(rel[:, k]))) for k, lab in enumerate(labels)))
    # inside the staging function (workgroup 101, layer 2): six stamps per phase, relative to the moment the last
    # workgroup finished the epilogue of the phase before
    if n_layers >= 3 and n_wg > 101:
        fine = buf[n_wg * 64 + 512:n_wg * 64 + 512 + 32].reshape(4, 8)
        t0 = tl[:, 0].min()
        before = {"qkv": "w2 fin l1", "wo": "qkv fin l2", "w13": "wo fin l2", "w2": "w13 fin l2"}
        for k, ph in enumerate(PHASES):
            # (a vector that is normalised has a barrier of its own after the wait; one that is only quantised has not)
            labels = (("entered", "first poll back", "its words there", "all wavefronts' there", "its blocks quantised",
                       "all quantised") if ph in ("qkv", "w13") else
                      ("entered", "first poll back", "its words there", "its blocks quantised", "all quantised"))
            last = float(us[:, names.index(before[ph])].max())
            f = (fine[k][:len(labels)] - t0) * 0.01 - last
            print("staging for %-3s (workgroup 101, layer 2), us after the last workgroup's previous epilogue: " % ph +
                  ", ".join("%s %+.2f" % (lab, float(v)) for lab, v in zip(labels, f)))
        # the end of every wavefront's streaming loop in that workgroup and layer, relative to the drained stamp of the phase
        # (the moment the loops start); the all-q4_K loop only
        waves = buf[n_wg * 64 + 600:n_wg * 64 + 600 + 64].reshape(4, 16)
        for k, ph in enumerate(PHASES):
            if waves[k].min() <= 0:
                continue
            start = float(us[101, names.index("%s drained l2" % ph)])
            w = (waves[k] - t0) * 0.01 - start
            print("loop of %-3s (workgroup 101, layer 2), us after the loops started, wavefronts 0..15: " % ph +
                  " ".join("%.2f" % float(v) for v in w))
    dev.close()


if __name__ == "__main__":
    main()
