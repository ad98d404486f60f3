"""Operator case directories in the layout of the reference's operator test
(tests/test_op.cc:399-447 file readers, :479-660 the replay loop):

    <root>/<op_name>/<case>/attr.txt     one line: JSON dict of string attributes
                            in_<i>.txt   input i:  "ndim d0 .. d(ndim-1) v0 v1 ..." (whitespace separated)
                            out_<i>.txt  expected output i, same format
                            err.txt      non-empty first line: shape inference must reject the case

`replay_case` does for one directory what the reference's loop does: count the
in_/out_ files, infer the output shapes (a failure is correct exactly when
err.txt announces one), compare the number and shapes of the outputs, run the
operator and compare every value.  The operator runs on the GPU through
CVMHIPRunOp; there is no host fallback.

    python cvm-runtime_amd/op_cases.py <root> [op ...]
"""
import json
import os
import sys

import numpy as np


def read_tensor(path):
    with open(path) as f:
        tok = f.read().split()
    ndim = int(tok[0])
    shape = tuple(int(t) for t in tok[1:1 + ndim])
    size = int(np.prod(shape, dtype=np.int64)) if ndim else 1
    vals = np.array([int(t) for t in tok[1 + ndim:1 + ndim + size]], dtype=np.int64)
    if vals.size != size:
        raise ValueError("%s: %d values for shape %s" % (path, vals.size, shape))
    return vals.astype(np.int32).reshape(shape)


def write_tensor(path, a):
    a = np.asarray(a)
    with open(path, "w") as f:
        f.write("%d\n" % a.ndim)
        f.write(" ".join(str(int(d)) for d in a.shape) + "\n")
        f.write(" ".join(str(int(v)) for v in a.ravel()) + "\n")


def _first_line(path):
    if not os.path.exists(path):
        return ""
    with open(path) as f:
        return f.readline().strip()


def read_case(path):
    names = os.listdir(path)
    n_in = sum(1 for n in names if n.startswith("in_"))
    n_out = sum(1 for n in names if n.startswith("out_"))
    return {"attrs": json.loads(_first_line(os.path.join(path, "attr.txt")) or "{}"),
            "ins": [read_tensor(os.path.join(path, "in_%d.txt" % i)) for i in range(n_in)],
            "outs": [read_tensor(os.path.join(path, "out_%d.txt" % i)) for i in range(n_out)],
            "err": _first_line(os.path.join(path, "err.txt"))}


def write_case(path, attrs, ins, outs, err=""):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "attr.txt"), "w") as f:
        f.write(json.dumps(attrs) + "\n")
    for i, v in enumerate(ins):
        write_tensor(os.path.join(path, "in_%d.txt" % i), v)
    for i, v in enumerate(outs):
        write_tensor(os.path.join(path, "out_%d.txt" % i), v)
    with open(os.path.join(path, "err.txt"), "w") as f:
        f.write(err + ("\n" if err else ""))


def list_cases(root, ops=None):
    found = []
    for op in sorted(os.listdir(root)):
        d = os.path.join(root, op)
        if not os.path.isdir(d) or (ops and op not in ops):
            continue
        for case in sorted(os.listdir(d)):
            if os.path.isdir(os.path.join(d, case)):
                found.append((op, os.path.join(d, case)))
    return found


def replay_case(op, path, run_op=None, execute=True):
    """(ok, detail) for one case directory.  `run_op` defaults to the GPU library's
    single-operator call; execute=False stops after shape inference (no GPU)."""
    if run_op is None:
        from . import runtime
        run_op = runtime.run_op
    case = read_case(path)
    rc, stage, outs, msg = run_op(op, case["attrs"], case["ins"], execute=False)
    if rc != 0:
        if case["err"]:
            return True, "rejected as announced: " + msg.splitlines()[0][:120]
        return False, "shape inference failed: " + msg
    if case["err"]:
        return False, "err.txt announces '%s' but shape inference accepted the case" % case["err"]
    if len(outs) != len(case["outs"]):
        return False, "should be %d outputs but we calculated %d" % (len(case["outs"]), len(outs))
    for i, (o, want) in enumerate(zip(outs, case["outs"])):
        if o.shape != want.shape:
            return False, "output %d: shape %s, expected %s" % (i, o.shape, want.shape)
    if not execute:
        return True, "shapes agree"
    rc, stage, outs, msg = run_op(op, case["attrs"], case["ins"])
    if rc != 0:
        return False, "operator failed (status %d): %s" % (rc, msg)
    for i, (o, want) in enumerate(zip(outs, case["outs"])):
        if not np.array_equal(o, want):
            bad = np.flatnonzero(o.ravel() != want.ravel())
            return False, "output %d: %d of %d values differ, first at %d: got %d, expected %d" % (
                i, bad.size, want.size, bad[0], o.ravel()[bad[0]], want.ravel()[bad[0]])
    return True, "match"


def replay_tree(root, ops=None, run_op=None, execute=True, log=None):
    results = []
    for op, path in list_cases(root, ops):
        ok, detail = replay_case(op, path, run_op, execute)
        results.append((op, path, ok, detail))
        if log:
            log("match %d | %s %s: %s" % (ok, op, os.path.basename(path), detail))
    return results


def main(argv):
    if len(argv) < 2:
        sys.exit(__doc__)
    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.dirname(here))
    import __graft_entry__
    pkg = __graft_entry__.load_package()
    from cvm_runtime_amd import op_cases
    res = op_cases.replay_tree(argv[1], set(argv[2:]) or None, log=print)
    bad = [r for r in res if not r[2]]
    print("%d cases, %d failed" % (len(res), len(bad)))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
