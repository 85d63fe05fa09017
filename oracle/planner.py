"""Oracle: the forward-request planner (integer page-table logic).  TEST INFRASTRUCTURE ONLY.

Restates, in plain Python integers, what the reference's portable driver derives from the
wire arrays of a forward request:
  seq_len            driver/portable/src/plan.cpp:247-249
  physical slot      driver/portable/src/plan.hpp:36-45  (page_indices[off + pos//ps]*ps + pos%ps)
  visible keys       driver/portable/src/plan.cpp:54-94  (j <= min(n_kv-1, pos))
  sampling rows      driver/portable/src/plan.cpp:355-373 (qo_start + relative index)
  shape/range checks driver/portable/src/plan.cpp:177-206, :236-287
  pure decode        driver/portable/src/executor/executor.cpp:537-543
Pinned by tests/test_planner.py against the wire-layout known answers of
runtime/src/inference/request.rs:810-897 and brute force over tiny page tables.
"""
from __future__ import annotations


class PlanError(ValueError):
    pass


def physical_idx(page_indices, off: int, page_size: int, pos: int) -> int:
    return int(page_indices[off + pos // page_size]) * page_size + pos % page_size


def plan_forward(token_ids, position_ids, kv_page_indices, kv_page_indptr, kv_last_page_lens,
                 qo_indptr, sampling_indices, sampling_indptr, page_size: int, total_pages: int,
                 num_samplers=None):
    R = len(qo_indptr) - 1
    if R <= 0:
        raise PlanError("plan: no requests in batch")
    if len(token_ids) != len(position_ids):
        raise PlanError("plan: token_ids/position_ids size mismatch")
    if len(kv_page_indptr) != R + 1:
        raise PlanError("plan: kv_page_indptr length must be num_requests+1")
    if len(kv_last_page_lens) != R:
        raise PlanError("plan: kv_last_page_lens length must equal num_requests")
    if len(sampling_indptr) != R + 1:
        raise PlanError("plan: sampling_indptr length must be num_requests+1")
    N = len(token_ids)
    out = dict(R=R, N=N, positions=[0] * N, kv_slots=[0] * N, row_page_begin=[0] * N,
               row_kv_len=[0] * N, seq_len=[0] * R, sample_rows=[], sample_indptr=[0],
               max_kv_len=0, pure_decode=True)
    for r in range(R):
        qs, qe = int(qo_indptr[r]), int(qo_indptr[r + 1])
        if qe - qs <= 0:
            raise PlanError(f"plan: request {r} has zero tokens")
        if qe - qs != 1:
            out["pure_decode"] = False
        off = int(kv_page_indptr[r])
        npg = int(kv_page_indptr[r + 1]) - off
        seq = (npg - 1) * page_size + int(kv_last_page_lens[r]) if npg > 0 else 0
        if seq <= 0:
            raise PlanError(f"plan: request {r} has empty KV state")
        out["seq_len"][r] = seq
        for pi in range(npg):
            if int(kv_page_indices[off + pi]) >= total_pages:
                raise PlanError(f"plan: page id {int(kv_page_indices[off + pi])} out of bounds "
                                f"(total_pages={total_pages})")
        for i in range(qs, qe):
            pos = int(position_ids[i])
            if pos >= seq:
                raise PlanError(f"plan: request {r} token at position {pos} exceeds seq_len {seq}")
            out["positions"][i] = pos
            out["kv_slots"][i] = physical_idx(kv_page_indices, off, page_size, pos)
            out["row_page_begin"][i] = off
            out["row_kv_len"][i] = min(seq, pos + 1)
            out["max_kv_len"] = max(out["max_kv_len"], out["row_kv_len"][i])
        ss, se = int(sampling_indptr[r]), int(sampling_indptr[r + 1])
        for k in range(ss, se):
            rel = int(sampling_indices[k])
            if rel < 0 or rel >= qe - qs:
                raise PlanError(f"plan: request {r} sampling_index {rel} out of relative [0,{qe - qs})")
            out["sample_rows"].append(qs + rel)
        out["sample_indptr"].append(len(out["sample_rows"]))
    return out
