"""Graph descriptions as dictionaries, and their hand-over to the tim::vx C++ runtime.

A graph is ``{"test": name, "tensors": [...], "ops": [...], "output": tensor id}`` with
tensors ``{"id", "dtype", "attr", "shape", "quant": {"type", "channel_dim", "scales",
"zero_points"}, "data"}`` (shape in the API's order, dimension 0 fastest; data a list, a
``{"fill", "n"}`` record, a numpy array or None) and operators ``{"kind", "inputs",
"outputs", "attrs"}``. `write_graphs` serialises such graphs into the text + blob pair the
`tvx_graph_runner` tool reads; `run_graphs` runs the tool, which builds every graph through
the public tim::vx API (Context / Graph / Tensor / ops::*), and returns what each produced.
"""
import os
import subprocess

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
RUNNER = os.path.join(PKG_DIR, "lib", "tvx_graph_runner")

NP_DTYPE = {"UINT8": np.uint8, "INT8": np.int8, "INT16": np.int16, "INT32": np.int32,
            "UINT32": np.uint32, "FLOAT16": np.float16, "FLOAT32": np.float32}

NO_QUANT = {"type": "NONE", "channel_dim": -1, "scales": [], "zero_points": []}


def asym(scale, zp):
    return {"type": "ASYMMETRIC", "channel_dim": -1, "scales": [float(scale)], "zero_points": [int(zp)]}


def sym_per_channel(scales, channel_dim):
    return {"type": "SYMMETRIC_PER_CHANNEL", "channel_dim": int(channel_dim),
            "scales": [float(s) for s in scales], "zero_points": [0] * len(scales)}


def tensor(tid, dtype, attr, shape, quant=None, data=None):
    return {"id": tid, "dtype": dtype, "attr": attr, "shape": [int(d) for d in shape],
            "quant": quant or NO_QUANT, "data": data}


_DEFAULT_ATTRS = {"pad_type": "AUTO", "pad": [0, 0, 0, 0], "stride": [1, 1], "dilation": [1, 1],
                  "ksize": [0, 0], "multiplier": 0, "weights": 0, "pool_type": "MAX",
                  "round_type": "FLOOR", "pool_1d": False, "axis": 0, "beta": 1.0, "sm_axis": 0,
                  "new_shape": [], "groups": 0, "conv_1d": False, "perm": [],
                  "layout": "ANY", "kernel_layout": "ANY", "output_padding": [0, 0]}


# "pool_1d": False / True, or the Pool2d constructor to call: "global" (ksize = input size) or "adaptive"
# (ksize = input size, stride = output size)
_POOL_FORM = {False: 0, True: 1, 0: 0, 1: 1, "global": 2, "adaptive": 3}


def op(kind, inputs, outputs, **attrs):
    a = dict(_DEFAULT_ATTRS)
    a.update(attrs)
    return {"kind": kind, "inputs": list(inputs), "outputs": list(outputs), "attrs": a}


def tensor_bytes(t):
    """Raw little-endian bytes of a tensor's data, or b'' when it has none."""
    d = t["data"]
    if d is None:
        return b""
    dt = NP_DTYPE[t["dtype"]]
    if isinstance(d, dict):
        return np.full(int(d["n"]), d["fill"], dtype=dt).tobytes()
    return np.ascontiguousarray(np.asarray(d).astype(dt, copy=False)).tobytes()


def write_graphs(graphs, txt_path, blob_path, bench=None):
    """bench = (warmup, iters) adds a timing record after each graph's run."""
    off = 0
    with open(txt_path, "w") as txt, open(blob_path, "wb") as blob:
        for g in graphs:
            txt.write("graph %s\n" % g["test"].replace(" ", "_"))
            if g.get("handles"):
                txt.write("handles\n")
            if g.get("platform"):
                txt.write("platform\n")
            if g.get("device") is not None:
                txt.write("device %d\n" % g["device"])
            if g.get("clone"):
                txt.write("clone\n")
            for t in g["tensors"]:
                raw = tensor_bytes(t)
                q = t["quant"]
                f = ["t", t["id"], t["dtype"], t["attr"], len(t["shape"])] + list(t["shape"])
                f += [q["type"], q["channel_dim"], len(q["scales"])] + ["%.9g" % s for s in q["scales"]]
                f += [len(q["zero_points"])] + list(q["zero_points"]) + [off, len(raw)]
                txt.write(" ".join(str(x) for x in f) + "\n")
                blob.write(raw)
                off += len(raw)
            for o in g["ops"]:
                a = dict(_DEFAULT_ATTRS)
                a.update(o["attrs"])
                f = ["op", o["kind"], len(o["inputs"])] + list(o["inputs"]) + [len(o["outputs"])] + list(o["outputs"])
                f += [a["pad_type"]] + list(a["pad"]) + list(a["stride"]) + list(a["dilation"]) + list(a["ksize"])
                f += [a["multiplier"], a["weights"], a["pool_type"], a["round_type"], _POOL_FORM[a["pool_1d"]],
                      a["axis"], "%.9g" % a["beta"], a["sm_axis"], len(a["new_shape"])] + list(a["new_shape"]) + [a["groups"], int(bool(a["conv_1d"]))]
                f += [len(a["perm"])] + list(a["perm"]) + [a["layout"], a["kernel_layout"]] + list(a["output_padding"])
                txt.write(" ".join(str(x) for x in f) + "\n")
            if g.get("layout_inference"):
                txt.write("infer\n")
            txt.write("run %d\n" % g["output"])
            # optional re-runs of the compiled graph with other input data: [{tensor id: array}, ...]
            dtypes = {t["id"]: NP_DTYPE[t["dtype"]] for t in g["tensors"]}
            for feeds in g.get("reruns", []):
                for tid, data in feeds.items():
                    raw = np.ascontiguousarray(np.asarray(data).astype(dtypes[tid], copy=False)).tobytes()
                    txt.write("feed %d %d %d\n" % (tid, off, len(raw)))
                    blob.write(raw)
                    off += len(raw)
                txt.write("run %d\n" % g["output"])
            if bench:
                txt.write("bench %d %d\n" % bench)
            txt.write("end\n")


def run_graphs(graphs, workdir, bench=None, timeout=600, env=None, threads=0, lock=True):
    """Returns (outputs, info, log): per graph the flat output array (None where the runtime
    refused the graph, the stage then in info[name]["fail"]); with `bench`, info[name] holds
    the milliseconds per Graph::Run() as "run_ms" (whole call, host copies included) and
    "device_ms" (the operator sequence alone); a graph with "reruns" (a list of {input tensor
    id: data}) is run again once per entry and info[name]["reruns"] lists those outputs; log is
    what the runtime wrote to stderr. With `threads` the runner processes the file in that many threads (one after
    the other under one mutex, or all at once with lock=False), each from Context::Create() on; it fails unless all
    threads produce the same bytes, and the first thread's results are returned."""
    if not os.path.exists(RUNNER):
        raise RuntimeError("%s is not built: run build.py" % RUNNER)
    os.makedirs(workdir, exist_ok=True)
    txt, blob, out = (os.path.join(workdir, n) for n in ("graphs.txt", "blob.bin", "out.bin"))
    write_graphs(graphs, txt, blob, bench)
    e = dict(os.environ)
    e.update(env or {})
    cmd = [RUNNER, txt, blob, out]
    if threads:
        cmd = [RUNNER, "--threads", str(threads)] + ([] if lock else ["--no-lock"]) + [txt, blob, out]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=timeout, env=e)
    if p.returncode != 0:
        raise RuntimeError("tvx_graph_runner exit %d\n%s\n%s" % (p.returncode, p.stdout[-2000:], p.stderr[-4000:]))
    raw = open(out + ".0" if threads else out, "rb").read()
    results, info = [], {}
    by_name = {}
    for line in p.stdout.splitlines():
        f = line.split()
        if not f:
            continue
        if f[0] == "ok":
            by_name.setdefault(f[1], []).append((int(f[2]), int(f[3])))
        elif f[0] == "fail":
            by_name.setdefault(f[1], []).append(None)
            info.setdefault(f[1], {})["fail"] = f[2]
        elif f[0] == "bench":
            info.setdefault(f[1], {}).update(run_ms=float(f[2]), device_ms=float(f[3]))
        elif f[0] == "opbench":  # per-operator device time (env TVX_RUNTIME_PROFILE=ops)
            info.setdefault(f[1], {}).setdefault("ops_us", []).append((f[3], float(f[4])))
            if len(f) > 5:  # the bytes of the operator's operands and result
                info[f[1]].setdefault("ops_bytes", []).append(int(f[5]))
    cursor = {}
    for g in graphs:
        name = g["test"].replace(" ", "_")
        i = cursor.get(name, 0)
        n_runs = 1 + len(g.get("reruns", []))
        cursor[name] = i + n_runs
        recs = by_name.get(name, [])[i:i + n_runs]
        recs += [None] * (n_runs - len(recs))
        t = {t["id"]: t for t in g["tensors"]}[g["output"]]
        arrays = [None if r is None else np.frombuffer(raw[r[0]:r[0] + r[1]], dtype=NP_DTYPE[t["dtype"]]).copy()
                  for r in recs]
        results.append(arrays[0])
        if n_runs > 1:
            info.setdefault(name, {})["reruns"] = arrays[1:]
    return results, info, p.stderr
