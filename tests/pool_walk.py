"""A seeded walk of the pool (alloc / free / empty_cache / the other tenant claiming and returning pages) run on
the C++ pool through the C ABI and on oracle.host.PoolModel side by side: after every operation the offset handed
out, the bytes released, the owner of EVERY physical page, the slot every page is mapped at and the bytes in use
must agree.  Shared by the CPU test (the pool's CPU backend) and the GPU test (the HIP virtual-memory backend)."""
import ctypes
import random

from oracle.host import PoolModel

MB = 1 << 20
SIZES = [512, 4096, 100_000, MB, 2 * MB - 1024, 2 * MB, 3 * MB, 20 * MB, 40 * MB, 70 * MB]


def walk_against_model(L, seed, pool_mb, page_mb, lazy, use_gpu, steps=600):
    """Returns (allocations that succeeded, allocations refused) -- both sides refuse the same ones."""
    assert L.tch_pool_init_ex(0, pool_mb * MB, int(use_gpu), page_mb * MB, int(lazy)) == 0, L.tch_host_last_error()
    model = PoolModel(pool_mb * MB, page_mb * MB, bool(lazy))
    rng = random.Random(seed)
    live, ok, refused = [], 0, 0
    n = model.n_pages
    owner, slot = (ctypes.c_uint8 * n)(), (ctypes.c_int64 * n)()
    try:
        for step in range(steps):
            r = rng.random()
            if r < 0.5 or not live:
                size = rng.choice(SIZES)
                ptr, want = L.tch_pool_malloc(size, 0, None), model.alloc(size)
                got = L.tch_pool_offset_of(0, ptr) if ptr else None
                assert got == want, f"step {step}: alloc({size}) at {got}, model {want}"
                if ptr:
                    live.append((ptr, want))
                    ok += 1
                else:
                    refused += 1
            elif r < 0.85:
                ptr, off = live.pop(rng.randrange(len(live)))
                L.tch_pool_free(ptr, 0, 0, None)
                model.free(off)
            elif r < 0.92:
                got, want = L.tch_cuda_memory_pool_free_train_local(0), model.empty_cache()
                assert got == want, f"step {step}: empty_cache released {got}, model {want}"
            elif r < 0.96:
                k = rng.randrange(1, 6)
                assert L.tch_pool_infer_claim_pages(0, k) == model.infer_claim(k), step
            else:
                k = rng.randrange(1, 6)
                assert L.tch_pool_infer_release_pages(0, k) == model.infer_release(k), step
            assert L.tch_pool_page_table(0, owner, slot, n) == n
            assert list(owner) == model.owner, f"step {step}: page owners differ"
            page_slot = {p: s for s, p in model.slot_page.items()}
            assert list(slot) == [page_slot.get(i, -1) for i in range(n)], f"step {step}: page placement differs"
            assert L.tch_cuda_memory_pool_train_usage(0) == model.train_usage, step
            assert L.tch_cuda_memory_pool_num_free_pages(0) == model.free_pages(), step
            assert L.tch_cuda_memory_pool_train_all_usage(0) == model.train_pages() * page_mb * MB, step
        for ptr, off in live:
            L.tch_pool_free(ptr, 0, 0, None)
            model.free(off)
        assert L.tch_cuda_memory_pool_free_train_local(0) == model.empty_cache()
        assert L.tch_cuda_memory_pool_train_all_usage(0) == 0 == model.train_pages()
    finally:
        L.tch_pool_shutdown(0)
    return ok, refused
