"""Child process of tests/test_gpu_xcc_exchange.py: runs sparse-layer launches under the value of
TIDAL_XCC_LOCAL it was started with and prints one JSON line with what it saw.  (The library probes
the device's workgroup placement once per process, so each setting needs a process of its own.)"""
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from _util import ATOL, PagedCase, randn, rotated, tolerance_report  # noqa: E402

TICKET_SLOTS, SLOT_BYTES = 15360, 64


def main():
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    cuda = torch.device("cuda:0")
    out = {"cases": []}
    for name, hq, hkv, rows, dtype, ks, fused in (
            ("mha", 32, 32, 32, torch.bfloat16, (2048, 2048, 600, 2048), False),
            ("mha-fused", 16, 16, 16, torch.float16, (1500, 1500, 1500), True),
            ("gqa-shared", 32, 8, 8, torch.bfloat16, (4096, 4096, 700), False),
            ("gqa-shared-fused", 32, 8, 8, torch.float16, (1024, 1024), True)):
        d, page, n = 128, 16, 6000
        case = PagedCase(n, hkv, d, page, dtype, seed=len(name))
        pool = case.pool.to(cuda)
        q = randn((hq, d), 3, dtype)
        w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
        w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))
        g = torch.Generator().manual_seed(1)
        worst, names = 0.0, []
        for k in ks:
            pos = torch.stack([torch.randperm(n - 1, generator=g)[:k] for _ in range(rows)])
            qd = q.to(dtype).to(cuda)[None]
            od = torch.full_like(qd, float("nan"))
            if fused:
                pos[:, -1] = n - 1
                theta = 1e4
                k_new, v_new = randn((1, hkv, d), 7, dtype), randn((1, hkv, d), 8, dtype)
                kk, vv = case.k.clone(), case.v.clone()
                kk[n - 1] = rotated(k_new, [n - 1], dtype, theta)[0]
                vv[n - 1] = v_new[0]
                want = orc.sparse_layer_gather(rotated(q[None], [n - 1], dtype, theta)[0], kk, vv, pos)
                cos, sin = _kernels.rope_table(torch.tensor([n - 1], dtype=torch.int32, device=cuda), d, 1.0, theta)
                dst = case.slots_of(torch.tensor([n - 1])).to(torch.int32).to(cuda)
                pl = pool.clone()
                w.forward(qd, od, pl, case.slots_of(pos).to(torch.int32).to(cuda), None, 0, 0, None,
                          index_kind="slots",
                          fresh=(k_new.to(dtype).to(cuda), v_new.to(dtype).to(cuda), cos, sin, dst))
            else:
                want = orc.sparse_layer_gather(q, case.k, case.v, pos)
                w.forward(qd, od, pool, case.slots_of(pos).to(torch.int32).to(cuda), None, 0, 0, None,
                          index_kind="slots")
            torch.cuda.synchronize()
            worst = max(worst, tolerance_report(od[0], want) / ATOL[dtype])
            names.append(_kernels.last_decode_kernel())
        ws = w._workspace[: 1 << 20].view(torch.int32).cpu()
        slots = ws[: TICKET_SLOTS * SLOT_BYTES // 4].view(TICKET_SLOTS, SLOT_BYTES // 4)
        marks = ws[TICKET_SLOTS * SLOT_BYTES // 4: TICKET_SLOTS * SLOT_BYTES // 4 + TICKET_SLOTS]
        out["cases"].append({
            "name": name, "worst_error_over_tolerance": worst, "kernels": names,
            "marked_slots": marks.nonzero().flatten().tolist(),
            "memory_tickets_nonzero": slots[:, 0].nonzero().flatten().tolist(),
            "l2_tickets_nonzero": slots[:, 1].nonzero().flatten().tolist(),
            "heads_per_row": hq // rows if rows == hkv and hq != hkv else 1, "rows": rows})
    print(json.dumps(out))


if __name__ == "__main__":
    main()
