"""ctypes front end of oracle/_ref/libpie_ref.so: the reference's own host sampler
(driver/portable/src/sampler.cpp) and BRLE decoder (driver/cuda/src/brle.cpp), compiled from the
reference tree by oracle/build_ref.py.  TEST INFRASTRUCTURE ONLY: tests use it to pin the oracle's
restatement (oracle/src/sampler.c, orc_brle_allow) and to measure how often the GPU samplers'
tokens differ from the reference's own.  `lib()` returns None where neither the library nor the
reference tree exists."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import build_ref

_lib = None
_tried = False

# the reference's SamplerType values (sampler.hpp) by the names the oracle uses
REF_TYPE = {"multinomial": 1, "top_k": 2, "top_p": 3, "min_p": 4, "top_k_top_p": 5}


def lib():
    global _lib, _tried
    if not _tried:
        _tried = True
        path = build_ref.build()
        if path is not None and path.exists():
            _lib = C.CDLL(str(path))
            _lib.ref_brle_decode.restype = C.c_long
    return _lib


def _p(a):
    return None if a is None else C.c_void_p(a.ctypes.data)


def _u32(a):
    return np.ascontiguousarray(np.asarray(a, np.uint32))


def sample_token(logits_f32, kind: str, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, seed=1) -> int:
    """sample_token (sampler.cpp:345-409) with the uniform drawn from Pcg32(seed)."""
    lg = np.ascontiguousarray(np.asarray(logits_f32, np.float32))
    tok = C.c_uint32(0)
    rc = lib().ref_sample_token(_p(lg), C.c_int(lg.size), C.c_int(REF_TYPE[kind]), C.c_float(temperature),
                                C.c_uint32(top_k), C.c_float(top_p), C.c_float(min_p), C.c_uint32(seed),
                                C.byref(tok))
    if rc != 0:
        raise RuntimeError("the reference's sample_token threw")
    return int(tok.value)


def distribution(logits_f32, temperature: float, k: int):
    lg = np.ascontiguousarray(np.asarray(logits_f32, np.float32))
    ids = np.empty(lg.size, np.uint32)
    vals = np.empty(lg.size, np.float32)
    n = lib().ref_distribution(_p(lg), C.c_int(lg.size), C.c_float(temperature), C.c_uint32(k), _p(ids), _p(vals))
    if n < 0:
        raise RuntimeError("the reference's sample_slot threw")
    return ids[:n].copy(), vals[:n].copy()


def logprobs_at(logits_f32, labels) -> np.ndarray:
    lg = np.ascontiguousarray(np.asarray(logits_f32, np.float32))
    lb = _u32(labels)
    out = np.empty(lb.size, np.float32)
    if lib().ref_logprobs(_p(lg), C.c_int(lg.size), _p(lb), C.c_int(lb.size), _p(out)) != lb.size:
        raise ValueError("the reference's sample_slot threw (label outside the vocabulary?)")
    return out


def entropy(logits_f32) -> float:
    lg = np.ascontiguousarray(np.asarray(logits_f32, np.float32))
    h = C.c_float(0)
    if lib().ref_entropy(_p(lg), C.c_int(lg.size), C.byref(h)) != 0:
        raise RuntimeError("the reference's sample_slot threw")
    return float(h.value)


def sample_token_from_topk(top_idx, top_probs, kind: str, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0,
                           seed=1) -> int:
    """sample_token_from_topk (sampler.cpp:411-): the host finalize of the reference's batch
    shortcut over a descending top-K list of softmaxed probabilities."""
    idx = np.ascontiguousarray(np.asarray(top_idx, np.int32))
    pr = np.ascontiguousarray(np.asarray(top_probs, np.float32))
    tok = C.c_uint32(0)
    rc = lib().ref_sample_token_from_topk(_p(idx), _p(pr), C.c_int(idx.size), C.c_int(REF_TYPE[kind]),
                                          C.c_float(temperature), C.c_uint32(top_k), C.c_float(top_p),
                                          C.c_float(min_p), C.c_uint32(seed), C.c_uint64(0), C.byref(tok))
    if rc != 0:
        raise RuntimeError("the reference's sample_token_from_topk threw")
    return int(tok.value)


def apply_brle_logit_mask(logits_f32, runs) -> np.ndarray:
    lg = np.array(logits_f32, np.float32, copy=True)
    r = _u32(runs)
    lib().ref_apply_brle_logit_mask(_p(lg), C.c_int(lg.size), _p(r), C.c_size_t(r.size))
    return lg


def _brle_args(masks, mask_indptr, qo_indptr, kv_page_indptr, kv_last_page_lens):
    m, mi, qo, kp, kl = map(_u32, (masks, mask_indptr, qo_indptr, kv_page_indptr, kv_last_page_lens))
    if m.size == 0:
        m = np.zeros(1, np.uint32)[:0]
    return m, mi, qo, kp, kl


def brle_is_pure_causal(masks, mask_indptr, qo_indptr, kv_page_indptr, kv_last_page_lens, page_size) -> bool:
    m, mi, qo, kp, kl = _brle_args(masks, mask_indptr, qo_indptr, kv_page_indptr, kv_last_page_lens)
    rc = lib().ref_brle_is_pure_causal(_p(m), C.c_size_t(m.size), _p(mi), C.c_size_t(mi.size), _p(qo), _p(kp),
                                       _p(kl), C.c_int(qo.size - 1), C.c_int(page_size))
    if rc < 0:
        raise RuntimeError("the reference's is_pure_causal threw")
    return bool(rc)


def brle_decode(masks, mask_indptr, qo_indptr, kv_page_indptr, kv_last_page_lens, page_size):
    """brle::decode: (packed bytes, per-request byte offsets [R + 1], pure_causal flag)."""
    m, mi, qo, kp, kl = _brle_args(masks, mask_indptr, qo_indptr, kv_page_indptr, kv_last_page_lens)
    R = qo.size - 1
    args = (_p(m), C.c_size_t(m.size), _p(mi), C.c_size_t(mi.size), _p(qo), _p(kp), _p(kl), C.c_int(R),
            C.c_int(page_size))
    n = lib().ref_brle_decode(*args, None, None, None)
    if n < 0:
        raise ValueError("the reference's decode threw (malformed mask layout)")
    packed = np.zeros(max(int(n), 1), np.uint8)
    indptr = np.zeros(R + 1, np.int32)
    pc = C.c_int(0)
    lib().ref_brle_decode(*args, _p(packed), _p(indptr), C.byref(pc))
    return packed[:n], indptr, bool(pc.value)
