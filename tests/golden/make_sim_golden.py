"""Writes tests/golden/sim_golden.json: what the reference's own NumPy simulator
returns for the bodies of tests/golden/sim_cases.py.

    python tests/golden/make_sim_golden.py [/root/reference]

Runs only where a checkout of the reference exists: it puts
<reference>/python on sys.path and imports hckernel.kernel_sim /
hckernel.kernel_api (pure Python on numpy, sympy, greenlet) without letting
Python write bytecode there.  Nothing of the reference is copied: the output
holds the cases' input-dependent results only (masks, values, dtype names,
exception names, repr text), a few KB.  tests/test_oracle_sim_golden.py holds
oracle.hcsim to this file; the file records the NumPy version it was made with,
because the behaviours recorded here are numpy.ma's.
"""
import os
import sys
import types

sys.dont_write_bytecode = True

import numpy as np                               # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

import sim_cases                                 # noqa: E402


def reference_api(root):
    sys.path.insert(0, os.path.join(root, "python"))
    import hckernel.kernel_api as ka
    import hckernel.kernel_sim as ks
    api = types.SimpleNamespace(**{k: getattr(ka, k) for k in dir(ka) if not k.startswith("__")})
    api.kernel = ks.kernel
    return api


if __name__ == "__main__":
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = sim_cases.run_all(reference_api(root))
    out["numpy_version"] = np.frombuffer(np.__version__.encode(), dtype=np.uint8)
    path = os.path.join(HERE, "sim_golden.json")
    sim_cases.dump(out, path)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "entries")
