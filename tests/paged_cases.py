"""Synthetic paged-KV batches shaped like the runtime's wire arrays (shared by CPU and GPU tests)."""
import numpy as np


def make_paged_batch(rng, ctx_lens, hk, d, ps, shared_prefix_tokens=0, shared_fraction=0.0,
                     extra_pages=3, std=1.0, f32_to_bf16=None):
    """Page pool = random permutation; a fraction of the requests list the same physical
    pages for their first `shared_prefix_tokens` tokens (a forked prefix)."""
    R = len(ctx_lens)
    npages_req = [(int(c) + ps - 1) // ps for c in ctx_lens]
    shared_pages = shared_prefix_tokens // ps
    n_shared_req = int(round(shared_fraction * R))
    sharers = [r for r in range(R) if ctx_lens[r] >= shared_prefix_tokens][:n_shared_req]
    total = sum(npages_req) - (max(len(sharers) - 1, 0)) * shared_pages if shared_pages else sum(npages_req)
    total += extra_pages
    perm = rng.permutation(total).astype(np.uint32)
    nxt = 0
    prefix = None
    if shared_pages and sharers:
        prefix = perm[nxt:nxt + shared_pages]
        nxt += shared_pages
    indices, indptr, last = [], [0], []
    for r in range(R):
        n = npages_req[r]
        if prefix is not None and r in sharers:
            own = perm[nxt:nxt + n - shared_pages]
            nxt += n - shared_pages
            pages = np.concatenate([prefix, own])
        else:
            pages = perm[nxt:nxt + n]
            nxt += n
        indices.append(pages)
        indptr.append(indptr[-1] + n)
        last.append(0 if n == 0 else int(ctx_lens[r]) - (n - 1) * ps)
    k = rng.standard_normal((total, ps, hk, d)).astype(np.float32) * std
    v = rng.standard_normal((total, ps, hk, d)).astype(np.float32) * std
    return dict(
        k_pages=f32_to_bf16(k), v_pages=f32_to_bf16(v),
        page_indices=(np.concatenate(indices) if indices else np.zeros(0)).astype(np.uint32),
        page_indptr=np.array(indptr, np.uint32), last_lens=np.array(last, np.uint32),
        num_pages=total, sharers=sharers)


def gather_rows(batch, r, ps):
    """Dense [kv_len, hk, d] K and V (uint16 bits) of request r, straight from the definition."""
    lo, hi = int(batch["page_indptr"][r]), int(batch["page_indptr"][r + 1])
    pages = batch["page_indices"][lo:hi]
    if len(pages) == 0:
        shp = (0,) + batch["k_pages"].shape[2:]
        return np.zeros(shp, np.uint16), np.zeros(shp, np.uint16)
    kv_len = (len(pages) - 1) * ps + int(batch["last_lens"][r])
    k = batch["k_pages"][pages].reshape((-1,) + batch["k_pages"].shape[2:])[:kv_len]
    v = batch["v_pages"][pages].reshape((-1,) + batch["v_pages"].shape[2:])[:kv_len]
    return k, v
