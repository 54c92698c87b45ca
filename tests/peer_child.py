"""The other process of the cross-process pool tests: attaches to a pool some trainer created, claims pages, maps
them, reads what the trainer left and writes its own pattern, gives the pages back.  Started through
multiprocessing's fork server (brought up before anything in the test session touches the GPU), so that no
process that has initialised the GPU ever forks or execs."""
import ctypes
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def claim_map_write(conn, port, n_pages, expect_value, write_value):
    """Claims n_pages FREE pages and maps each.  The pages hold fp32 data.  Every access goes through kernels of
    the library (an address mapped from a foreign dma-buf is device memory to a kernel, but not a pointer the HIP
    copy routines know): `mine += page; page = 0` (tch_grad_accumulate) brings a page's content into a tensor of
    this process, which is compared with expect_value (None = do not check), and `page += pattern` then leaves
    write_value in every element of the page.  Reports, waits for 'go', unmaps and gives everything back."""
    try:
        os.environ["SIRIUS_PORT"] = str(port)
        if ROOT not in sys.path:
            sys.path.insert(0, ROOT)
        import torch
        from sirius_amd import ops
        from sirius_amd._lib import check, lib
        L = lib()
        out = {"pid": os.getpid()}
        torch.cuda.set_device(0)
        ctx = ops.Context(torch.cuda.current_stream())
        t0 = time.perf_counter()
        if L.tch_pool_peer_attach(0) != 0:
            raise RuntimeError(L.tch_host_last_error().decode())
        page_bytes = L.tch_pool_peer_page_bytes(0)
        n = page_bytes // 4
        got = (ctypes.c_int * n_pages)()
        out["claimed"] = L.tch_pool_peer_claim(0, n_pages, got)
        t1 = time.perf_counter()
        pages = list(got)[:out["claimed"]]
        out["indices"] = pages
        # pages the creator handed back lazily are claimable before their old mapping is gone: how many, right now
        out["still_mapped_at_claim"] = L.tch_pool_peer_still_mapped(0, got, out["claimed"])
        ptrs = []
        for pg in pages:
            p = L.tch_pool_peer_map(0, pg)
            if not p:
                raise RuntimeError(L.tch_host_last_error().decode())
            ptrs.append(p)
        t2 = time.perf_counter()
        seen_ok, sample = True, []
        for p in ptrs:
            mine = torch.zeros(n, device="cuda")
            check(L.tch_grad_accumulate(ctx.handle, ctypes.c_void_p(mine.data_ptr()), ctypes.c_void_p(p), n), "read page")
            pattern = torch.full((n,), float(write_value), device="cuda")
            check(L.tch_grad_accumulate(ctx.handle, ctypes.c_void_p(p), ctypes.c_void_p(pattern.data_ptr()), n), "write page")
            ctx.synchronize()
            torch.cuda.synchronize()
            sample.append(float(mine[0]))
            if expect_value is not None:
                seen_ok = seen_ok and bool((mine == float(expect_value)).all())
        out["seen_ok"], out["seen_sample"] = seen_ok, sample[:4]
        t3 = time.perf_counter()
        out["attach_claim_ms"], out["map_ms"], out["rw_ms"] = (t1 - t0) * 1e3, (t2 - t1) * 1e3, (t3 - t2) * 1e3
        # a page this process does not own is refused by the creator
        foreign = next(i for i in range(L.tch_pool_peer_num_pages(0)) if i not in pages)
        out["foreign_page_refused"] = not L.tch_pool_peer_map(0, foreign)
        conn.send(out)
        conn.recv()   # 'go'
        back = (ctypes.c_int * len(pages))(*pages)
        released = L.tch_pool_peer_release(0, back, len(pages))
        L.tch_pool_peer_detach(0)
        conn.send({"released": released})
    except Exception as e:   # the parent must not hang on a child that failed
        conn.send({"error": repr(e)})
    finally:
        conn.close()
