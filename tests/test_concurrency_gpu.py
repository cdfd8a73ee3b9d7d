"""Several contexts at once: the reference runs a pool of workers, each with its own backend instance
(docs/concurrency.md:52-61, src/core/ggml_cpu_backend.h:202-204), so calls arrive from several host threads.
The library keeps no per-call state besides the per-device scratch; threads that use their own streams pass their
own workspaces.  Results must be the ones a single thread gets, and mi355x_last_error() is per thread."""
import threading

import numpy as np
import pytest
import torch

import oracle as ora
from cases import make_case
from crispasr_amd import ggml
from gpu_util import assert_parity, run_oracle, upload

pytestmark = pytest.mark.gpu


def _workspace_bytes(q, k, v, m, scale, kernel, n_splits):
    return ggml.flash_attn_workspace_size(q, k, v, m, scale, kernel=kernel, n_splits=n_splits)


def test_two_host_threads_on_their_own_streams_and_workspaces():
    specs = [
        (dict(seed=901, D=128, Nq=1, Nkv=1500, Hq=16, Hkv=4, B=2, ktype=ora.Q8_0), ggml.KERNEL_DECODE_MMA, 6),   # split-KV + merge
        (dict(seed=902, D=64, Nq=300, Nkv=520, Hq=4, ktype=ora.F32, mask="bias"), ggml.KERNEL_MMA, 0),          # K/V rounded to f16 in the workspace
    ]
    jobs = []
    for spec, kernel, ns in specs:
        case = make_case(**spec)
        q, k, v = upload(case["q"]), upload(case["k"]), upload(case["v"])
        m = upload(case["mask"]) if case["mask"] is not None else None
        nbytes = _workspace_bytes(q, k, v, m, case["scale"], kernel, ns)
        assert nbytes > 0
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        single = ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=kernel, n_splits=ns, workspace=ws).numpy_f32()
        assert_parity(single, run_oracle(case), str(spec))
        jobs.append((case, q, k, v, m, kernel, ns, ws, single))
    torch.cuda.synchronize()
    errors = []

    def worker(i):
        case, q, k, v, m, kernel, ns, ws, single = jobs[i]
        stream = torch.cuda.Stream()
        try:
            for it in range(40):
                out = ggml.flash_attn_ext(q, k, v, m, case["scale"], kernel=kernel, n_splits=ns, workspace=ws, stream=stream)
                stream.synchronize()
                if not np.array_equal(out.numpy_f32(), single):
                    errors.append((i, it, "result differs from the single-threaded one"))
                    return
            # an error in this thread is reported to this thread only
            bad = ggml.flash_attn_supports(q, k, upload(make_case(seed=903, D=128 if q.ne[0] == 64 else 64, Nq=1, Nkv=k.ne[1], Hq=k.ne[2])["v"]), None)
            if bad == ggml.OK or not ggml.lib().mi355x_last_error():
                errors.append((i, "contract violation not reported"))
        except Exception as e:                                   # noqa: BLE001 - reported below, with the thread's index
            errors.append((i, repr(e)))

    print("two host threads, 40 calls each", flush=True)
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors
