"""Run as a script by tests/test_gpu_streams.py in a process of its own: torch is
imported first, so this library binds to the HIP runtime torch loaded, and torch
tensors are passed straight to the C ABI (data_ptr, current stream)."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import torch  # noqa: E402  (first on purpose)
import numpy as np  # noqa: E402
import __graft_entry__ as entry  # noqa: E402
from oracle import spmm_oracle as so  # noqa: E402

pkg = entry.load_package()
assert torch.cuda.is_available() and pkg.device_count() >= 1
g = pkg.synthetic.cfg1()
N = 64
X = pkg.synthetic.dense_operand("cfg1", g.n_cols, N)
tX = torch.from_numpy(X).cuda()
tY = torch.full((g.n_rows, N), float("nan"), device="cuda")
stream = torch.cuda.current_stream().cuda_stream

op = pkg.AccelSpMM(g.indptr, g.indices, g.values, g.n_cols).preprocess()     # CSR uploaded from numpy
op.run(tX, tY, N, stream=stream)
torch.cuda.synchronize()
err1 = so.check(tY.cpu().numpy(), g.indptr, g.indices, g.values, X)

ip, ix, v = (torch.from_numpy(a).cuda() for a in (g.indptr, g.indices, g.values))   # CSR borrowed from torch
op2 = pkg.AccelSpMM(ip, ix, v, g.n_cols, device=True, n_rows=g.n_rows, nnz=g.nnz).preprocess()
tY.fill_(float("nan"))
op2.run(tX, tY, N, stream=stream)
torch.cuda.synchronize()
err2 = so.check(tY.cpu().numpy(), g.indptr, g.indices, g.values, X)

# the same product by torch itself, as a second opinion
A = torch.sparse_csr_tensor(ip.long(), ix.long(), v, size=(g.n_rows, g.n_cols))
ref = (A @ tX).cpu().numpy()
rel = float(np.max(np.abs(ref - tY.cpu().numpy())) / np.max(np.abs(ref)))
with open("/proc/self/maps") as f:
    runtimes = sorted({line.split()[-1] for line in f if "libamdhip64" in line})
print(f"RESULT err1={err1:.3e} err2={err2:.3e} rel_vs_torch={rel:.3e} runtimes={len(runtimes)}")
assert err1 <= so.TOL and err2 <= so.TOL and rel <= 1e-5 and len(runtimes) == 1
