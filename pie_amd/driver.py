"""ctypes binding of the `hip` driver flavour (`libpie_driver_hip.so`).

Mirrors `include/pie_driver_abi.h`: the descriptor structs the Pie runtime exchanges
with an in-process driver, the direct embedding API (`pie_hip_driver_*`) and the
`pie_driver_hip_run_inproc` serve loop.  The classes here play the runtime's side of the
boundary in tests and benchmarks (what `runtime/tests/common/mock_device.rs` does from
the other side); nothing here computes.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import Iterable, Optional, Sequence

import numpy as np

_PKG = Path(__file__).resolve().parent
DRIVER_LIB_PATH = _PKG / "libpie_driver_hip.so"
_lib = None


class DriverLibraryMissing(RuntimeError):
    pass


def _slice_type(ctype, name):
    return type(name, (C.Structure,), {"_fields_": [("ptr", C.POINTER(ctype)), ("len", C.c_size_t)]})


U8Slice = _slice_type(C.c_uint8, "U8Slice")
U32Slice = _slice_type(C.c_uint32, "U32Slice")
U64Slice = _slice_type(C.c_uint64, "U64Slice")
F32Slice = _slice_type(C.c_float, "F32Slice")


class AdapterBindingDesc(C.Structure):
    _fields_ = [("adapter_id", C.c_int64), ("seed", C.c_int64)]


class BrleDesc(C.Structure):
    _fields_ = [("buffer", U32Slice), ("total_size", C.c_uint64)]


class SamplerDesc(C.Structure):
    _fields_ = [("kind", C.c_uint8), ("temperature", C.c_float), ("seed", C.c_uint32),
                ("k", C.c_uint32), ("p", C.c_float), ("num_tokens", C.c_uint32),
                ("token_id", C.c_uint32), ("token_ids", U32Slice)]


BrleSlice = _slice_type(BrleDesc, "BrleSlice")
SamplerSlice = _slice_type(SamplerDesc, "SamplerSlice")
AdapterBindingSlice = _slice_type(AdapterBindingDesc, "AdapterBindingSlice")

_FWD_REQ_FIELDS = [
    ("token_ids", U32Slice), ("position_ids", U32Slice), ("kv_page_indices", U32Slice),
    ("kv_page_indptr", U32Slice), ("kv_last_page_lens", U32Slice), ("qo_indptr", U32Slice),
    ("rs_slot_ids", U32Slice), ("rs_slot_flags", U8Slice), ("masks", BrleSlice),
    ("mask_indptr", U32Slice), ("logit_masks", BrleSlice), ("logit_mask_indptr", U32Slice),
    ("sampling_indices", U32Slice), ("sampling_indptr", U32Slice), ("samplers", SamplerSlice),
    ("sampler_indptr", U32Slice), ("adapter_bindings", AdapterBindingSlice),
    ("spec_token_ids", U32Slice), ("spec_position_ids", U32Slice), ("spec_indptr", U32Slice),
    ("output_spec_flags", U8Slice), ("context_ids", U64Slice),
    ("single_token_mode", C.c_uint8), ("has_user_mask", C.c_uint8),
    ("image_indptr", U32Slice), ("image_grids", U32Slice), ("image_anchor_positions", U32Slice),
    ("image_pixels", U8Slice), ("image_pixel_indptr", U32Slice),
    ("image_mrope_positions", U32Slice), ("image_mrope_indptr", U32Slice),
    ("image_patch_positions", U32Slice), ("image_anchor_rows", U32Slice),
    ("audio_features", U8Slice), ("audio_feature_indptr", U32Slice),
    ("audio_anchor_rows", U32Slice), ("audio_indptr", U32Slice),
]


class ForwardRequestDesc(C.Structure):
    _fields_ = _FWD_REQ_FIELDS


class CopyRequestDesc(C.Structure):
    _fields_ = [("dir", C.c_uint8), ("srcs", U32Slice), ("dsts", U32Slice), ("resource", C.c_uint8)]


class AdapterRequestDesc(C.Structure):
    _fields_ = [("op", C.c_uint8), ("adapter_id", C.c_uint64), ("path", U8Slice)]


class RequestPayloadDesc(C.Structure):
    _fields_ = [("kind", C.c_uint8), ("forward", ForwardRequestDesc), ("copy", CopyRequestDesc),
                ("adapter", AdapterRequestDesc)]


class FrameDesc(C.Structure):
    _fields_ = [("driver_id", C.c_uint32), ("payload", RequestPayloadDesc)]


class ForwardResponseDesc(C.Structure):
    _fields_ = [
        ("num_requests", C.c_uint32), ("tokens_indptr", U32Slice), ("tokens", U32Slice),
        ("dists_req_indptr", U32Slice), ("dists_kv_indptr", U32Slice), ("dists_ids", U32Slice),
        ("dists_probs", F32Slice), ("logits_req_indptr", U32Slice),
        ("logits_byte_indptr", U32Slice), ("logits_bytes", U8Slice),
        ("logprobs_req_indptr", U32Slice), ("logprobs_val_indptr", U32Slice),
        ("logprobs_values", F32Slice), ("entropies_indptr", U32Slice), ("entropies", F32Slice),
        ("spec_indptr", U32Slice), ("spec_tokens", U32Slice), ("spec_positions", U32Slice),
        ("probe_wire_parse_us", C.c_uint32), ("probe_plan_us", C.c_uint32),
        ("probe_h2d_us", C.c_uint32), ("probe_kernel_launch_us", C.c_uint32),
        ("probe_sync_us", C.c_uint32), ("probe_response_build_us", C.c_uint32),
    ]


class StatusResponseDesc(C.Structure):
    _fields_ = [("status", C.c_int32)]


class ResponsePayloadDesc(C.Structure):
    _fields_ = [("kind", C.c_uint8), ("forward", ForwardResponseDesc), ("status", StatusResponseDesc)]


class ResponseFrameDesc(C.Structure):
    _fields_ = [("driver_id", C.c_uint32), ("aborted", C.c_uint8), ("payload", ResponsePayloadDesc)]


RECV_FN = C.CFUNCTYPE(C.c_int32, C.c_void_p, C.POINTER(C.POINTER(FrameDesc)), C.POINTER(C.c_uint32))
SEND_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_uint32, C.POINTER(ResponseFrameDesc))
READY_FN = C.CFUNCTYPE(None, C.c_char_p, C.c_void_p)


class InProcVTable(C.Structure):
    _fields_ = [("recv", RECV_FN), ("send_response", SEND_FN), ("ctx", C.c_void_p)]


REQ_FORWARD, REQ_COPY, REQ_ADAPTER, REQ_HEALTH = 0, 1, 2, 3
RESP_FORWARD, RESP_STATUS = 0, 1
SAMPLER_TOP_P = 2


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not DRIVER_LIB_PATH.exists():
            raise DriverLibraryMissing(
                f"{DRIVER_LIB_PATH} is not built; run `python -m pie_amd.build`")
        l = C.CDLL(str(DRIVER_LIB_PATH))
        l.pie_hip_driver_create.restype = C.c_void_p
        l.pie_hip_driver_create.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t]
        l.pie_hip_driver_destroy.argtypes = [C.c_void_p]
        l.pie_hip_driver_capabilities.restype = C.c_char_p
        l.pie_hip_driver_capabilities.argtypes = [C.c_void_p]
        l.pie_hip_driver_handle.argtypes = [C.c_void_p, C.POINTER(FrameDesc), C.POINTER(ResponseFrameDesc)]
        l.pie_hip_driver_generate.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                              C.c_int, C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
        l.pie_hip_driver_set_generate_divergence.argtypes = [C.c_void_p, C.c_uint32]
        l.pie_hip_driver_set_generate_divergence.restype = C.c_int
        l.pie_hip_driver_set_generate_sampler.argtypes = [C.c_void_p, C.c_int, C.c_float, C.c_uint32,
                                                          C.c_float, C.c_uint32]
        l.pie_hip_driver_export_tensor.restype = C.c_size_t
        l.pie_hip_driver_export_tensor.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t]
        l.pie_hip_driver_tensor_ptr.restype = C.c_void_p
        l.pie_hip_driver_tensor_ptr.argtypes = [C.c_void_p, C.c_char_p]
        l.pie_hip_driver_plan.restype = C.c_longlong
        l.pie_hip_driver_plan.argtypes = [C.POINTER(ForwardRequestDesc), C.c_int, C.c_int, C.c_void_p,
                                          C.c_void_p, C.c_size_t, C.c_char_p, C.c_size_t]
        l.pie_driver_hip_run_inproc.restype = C.c_int
        l.pie_driver_hip_run_inproc.argtypes = [C.c_int, C.POINTER(C.c_char_p), C.c_int, READY_FN,
                                                C.c_void_p, InProcVTable]
        l.pie_driver_hip_request_stop.restype = None
        _lib = l
    return _lib


# ---------------------------------------------------------------- frame construction
class ForwardFrame:
    """Builds a forward `FrameDesc` over numpy arrays it keeps alive (the runtime's role)."""

    def __init__(self, token_ids, position_ids, kv_page_indices, kv_page_indptr,
                 kv_last_page_lens, qo_indptr, sampling_indices=None, sampling_indptr=None,
                 samplers: Optional[Sequence[dict]] = None, sampler_indptr=None,
                 context_ids=None, masks: Optional[Sequence[Sequence[int]]] = None,
                 driver_id: int = 0, logit_masks: Optional[Sequence[Sequence[int]]] = None,
                 logit_mask_indptr=None, spec_token_ids=None, spec_position_ids=None,
                 spec_indptr=None):
        R = len(qo_indptr) - 1
        self._keep = []

        def u32(a):
            arr = np.ascontiguousarray(np.asarray(a, dtype=np.uint32))
            self._keep.append(arr)
            return U32Slice(arr.ctypes.data_as(C.POINTER(C.c_uint32)), arr.size)

        self.frame = FrameDesc()
        self.frame.driver_id = driver_id
        self.frame.payload.kind = REQ_FORWARD
        f = self.frame.payload.forward
        f.token_ids = u32(token_ids)
        f.position_ids = u32(position_ids)
        f.kv_page_indices = u32(kv_page_indices)
        f.kv_page_indptr = u32(kv_page_indptr)
        f.kv_last_page_lens = u32(kv_last_page_lens)
        f.qo_indptr = u32(qo_indptr)
        if sampling_indices is None:  # default: greedy-sample the last token of every request
            qo = np.asarray(qo_indptr, dtype=np.int64)
            sampling_indices = (qo[1:] - qo[:-1] - 1).astype(np.uint32)
            sampling_indptr = np.arange(R + 1, dtype=np.uint32)
        f.sampling_indices = u32(sampling_indices)
        f.sampling_indptr = u32(sampling_indptr)
        n_slots = len(sampling_indices)
        if samplers is None:
            samplers = [dict(kind=SAMPLER_TOP_P, temperature=0.0, p=1.0)] * n_slots
            sampler_indptr = np.asarray(sampling_indptr, dtype=np.uint32)
        arr = (SamplerDesc * max(len(samplers), 1))()
        for i, s in enumerate(samplers):
            arr[i].kind = s.get("kind", SAMPLER_TOP_P)
            arr[i].temperature = s.get("temperature", 0.0)
            arr[i].seed = s.get("seed", 0)
            arr[i].k = s.get("k", 0)
            arr[i].p = s.get("p", 1.0)
            arr[i].num_tokens = s.get("num_tokens", 0)
            arr[i].token_id = s.get("token_id", 0)
            if s.get("token_ids") is not None:
                arr[i].token_ids = u32(s["token_ids"])
        self._keep.append(arr)
        f.samplers = SamplerSlice(C.cast(arr, C.POINTER(SamplerDesc)), len(samplers))
        f.sampler_indptr = u32(sampler_indptr)
        if context_ids is None:
            context_ids = np.arange(R, dtype=np.uint64)
        cid = np.ascontiguousarray(np.asarray(context_ids, dtype=np.uint64))
        self._keep.append(cid)
        f.context_ids = U64Slice(cid.ctypes.data_as(C.POINTER(C.c_uint64)), cid.size)
        if masks is not None:
            marr = (BrleDesc * max(len(masks), 1))()
            for i, runs in enumerate(masks):
                marr[i].buffer = u32(runs)
                marr[i].total_size = int(np.sum(runs))
            self._keep.append(marr)
            f.masks = BrleSlice(C.cast(marr, C.POINTER(BrleDesc)), len(masks))
        if logit_masks is not None:   # one BRLE per entry; logit_mask_indptr partitions them per request
            larr = (BrleDesc * max(len(logit_masks), 1))()
            for i, runs in enumerate(logit_masks):
                larr[i].buffer = u32(runs)
                larr[i].total_size = int(np.sum(runs))
            self._keep.append(larr)
            f.logit_masks = BrleSlice(C.cast(larr, C.POINTER(BrleDesc)), len(logit_masks))
            f.logit_mask_indptr = u32(logit_mask_indptr)
        if spec_indptr is not None:
            f.spec_token_ids = u32(spec_token_ids)
            f.spec_position_ids = u32(spec_position_ids)
            f.spec_indptr = u32(spec_indptr)
        f.single_token_mode = 1 if len(token_ids) == R else 0


def copy_frame(direction: int, srcs: Iterable[int], dsts: Iterable[int], resource: int = 0):
    s = np.ascontiguousarray(np.asarray(list(srcs), dtype=np.uint32))
    d = np.ascontiguousarray(np.asarray(list(dsts), dtype=np.uint32))
    fr = FrameDesc()
    fr.payload.kind = REQ_COPY
    fr.payload.copy.dir = direction
    fr.payload.copy.resource = resource
    fr.payload.copy.srcs = U32Slice(s.ctypes.data_as(C.POINTER(C.c_uint32)), s.size)
    fr.payload.copy.dsts = U32Slice(d.ctypes.data_as(C.POINTER(C.c_uint32)), d.size)
    fr._keep = (s, d)
    return fr


def _u32_list(sl) -> list:
    return [sl.ptr[i] for i in range(sl.len)]


class ForwardResult:
    def __init__(self, resp: ResponseFrameDesc):
        fr = resp.payload.forward
        self.kind = resp.payload.kind
        self.num_requests = fr.num_requests
        self.tokens_indptr = _u32_list(fr.tokens_indptr)
        self.tokens = _u32_list(fr.tokens)
        self.other_indptr_lens = {
            "dists_req_indptr": fr.dists_req_indptr.len, "dists_kv_indptr": fr.dists_kv_indptr.len,
            "logits_req_indptr": fr.logits_req_indptr.len,
            "logits_byte_indptr": fr.logits_byte_indptr.len,
            "logprobs_req_indptr": fr.logprobs_req_indptr.len,
            "logprobs_val_indptr": fr.logprobs_val_indptr.len,
            "entropies_indptr": fr.entropies_indptr.len, "spec_indptr": fr.spec_indptr.len,
        }
        f32 = lambda sl: np.ctypeslib.as_array(sl.ptr, shape=(sl.len,)).copy() if sl.len else np.zeros(0, np.float32)
        self.dists_req_indptr = _u32_list(fr.dists_req_indptr)
        self.dists_kv_indptr = _u32_list(fr.dists_kv_indptr)
        self.dists_ids = _u32_list(fr.dists_ids)
        self.dists_probs = f32(fr.dists_probs)
        self.logits_req_indptr = _u32_list(fr.logits_req_indptr)
        self.logits_byte_indptr = _u32_list(fr.logits_byte_indptr)
        self.logits_bytes = C.string_at(fr.logits_bytes.ptr, fr.logits_bytes.len) if fr.logits_bytes.len else b""
        self.logprobs_req_indptr = _u32_list(fr.logprobs_req_indptr)
        self.logprobs_val_indptr = _u32_list(fr.logprobs_val_indptr)
        self.logprobs_values = f32(fr.logprobs_values)
        self.entropies_indptr = _u32_list(fr.entropies_indptr)
        self.entropies = f32(fr.entropies)
        self.probes = dict(plan=fr.probe_plan_us, h2d=fr.probe_h2d_us,
                           launch=fr.probe_kernel_launch_us, sync=fr.probe_sync_us,
                           build=fr.probe_response_build_us)

    def tokens_of(self, r: int) -> list:
        return self.tokens[self.tokens_indptr[r]:self.tokens_indptr[r + 1]]

    def dists_of(self, r: int) -> list:
        """[(ids, probs), ...] of request r, one pair per Distribution slot."""
        out = []
        for i in range(self.dists_req_indptr[r], self.dists_req_indptr[r + 1]):
            a, b = self.dists_kv_indptr[i], self.dists_kv_indptr[i + 1]
            out.append((np.asarray(self.dists_ids[a:b], np.uint32), self.dists_probs[a:b]))
        return out

    def logits_of(self, r: int) -> list:
        """f32 logits rows of request r's RawLogits slots."""
        out = []
        for i in range(self.logits_req_indptr[r], self.logits_req_indptr[r + 1]):
            a, b = self.logits_byte_indptr[i], self.logits_byte_indptr[i + 1]
            out.append(np.frombuffer(self.logits_bytes[a:b], np.float32))
        return out

    def logprobs_of(self, r: int) -> list:
        out = []
        for i in range(self.logprobs_req_indptr[r], self.logprobs_req_indptr[r + 1]):
            out.append(self.logprobs_values[self.logprobs_val_indptr[i]:self.logprobs_val_indptr[i + 1]])
        return out

    def entropies_of(self, r: int) -> list:
        return list(self.entropies[self.entropies_indptr[r]:self.entropies_indptr[r + 1]])


class Driver:
    """One driver instance (weights + KV pool on the GPU), driven synchronously."""

    def __init__(self, config_toml: str):
        err = C.create_string_buffer(1024)
        self._h = lib().pie_hip_driver_create(config_toml.encode(), err, len(err))
        if not self._h:
            raise RuntimeError(f"pie_hip_driver_create: {err.value.decode()}")

    def close(self):
        if self._h:
            lib().pie_hip_driver_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def capabilities(self) -> dict:
        import json

        return json.loads(lib().pie_hip_driver_capabilities(self._h).decode())

    def handle(self, frame) -> ResponseFrameDesc:
        fr = frame.frame if isinstance(frame, ForwardFrame) else frame
        out = ResponseFrameDesc()
        rc = lib().pie_hip_driver_handle(self._h, C.byref(fr), C.byref(out))
        if rc != 0:
            raise RuntimeError("pie_hip_driver_handle failed")
        return out

    def forward(self, frame: ForwardFrame) -> ForwardResult:
        return ForwardResult(self.handle(frame))

    def generate(self, prompt: Sequence[int], max_new: int, replicate: int = 1, warmup: int = 0):
        """Greedy generation harness; returns (tokens[replicate, max_new], timings dict).
        The first `warmup` decode steps are left out of the decode timings."""
        p = np.ascontiguousarray(np.asarray(prompt, dtype=np.uint32))
        out = np.zeros((replicate, max_new), np.uint32)
        tm = np.zeros(4, np.float64)
        err = C.create_string_buffer(1024)
        rc = lib().pie_hip_driver_generate(self._h, p.ctypes.data, len(p), max_new, replicate,
                                           warmup, out.ctypes.data, tm.ctypes.data, err, len(err))
        if rc != 0:
            raise RuntimeError(f"pie_hip_driver_generate: {err.value.decode()}")
        return out, dict(prefill_us=tm[0], decode_wall_us=tm[1], decode_device_us=tm[2],
                         decode_steps=int(tm[3]))

    def set_generate_divergence(self, stride: int) -> None:
        """Replica c of `generate` feeds (its last sampled token + c * stride) % vocab into every
        decode step: the rows of a decode batch then differ (0: identical replicas)."""
        if lib().pie_hip_driver_set_generate_divergence(self._h, stride) != 0:
            raise RuntimeError("pie_hip_driver_set_generate_divergence failed")

    def set_generate_sampler(self, kind: int, temperature: float, k: int = 0, p: float = 1.0,
                             seed: int = 1):
        """Token sampler `generate` attaches to its decode steps (default greedy)."""
        rc = lib().pie_hip_driver_set_generate_sampler(self._h, kind, C.c_float(temperature), k,
                                                       C.c_float(p), seed)
        if rc != 0:
            raise RuntimeError("pie_hip_driver_set_generate_sampler: bad arguments")

    def tensor_ptr(self, name: str) -> int:
        p = lib().pie_hip_driver_tensor_ptr(self._h, name.encode())
        if not p:
            raise KeyError(name)
        return int(p)

    def export_tensor(self, name: str, dtype) -> Optional[np.ndarray]:
        n = lib().pie_hip_driver_export_tensor(self._h, name.encode(), None, 0)
        if n == 0:
            return None
        arr = np.empty(n // np.dtype(dtype).itemsize, dtype=dtype)
        lib().pie_hip_driver_export_tensor(self._h, name.encode(), arr.ctypes.data, n)
        return arr


def snapshot_info(directory: str) -> dict:
    """Host-only: what the driver's snapshot reader sees in a Hugging Face checkpoint directory
    (config.json fields as the driver maps them, and every safetensors entry)."""
    import json

    out = C.create_string_buffer(8 << 20)
    err = C.create_string_buffer(1024)
    f = lib().pie_hip_driver_snapshot_info
    f.restype = C.c_longlong
    f.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t]
    n = f(directory.encode(), out, len(out), err, len(err))
    if n < 0:
        raise RuntimeError(f"pie_hip_driver_snapshot_info: {err.value.decode()}")
    return json.loads(out.value.decode())


def plan(frame: ForwardFrame, page_size: int, total_pages: int) -> dict:
    """Runs the driver's host-side planner (no GPU) and returns its integer plan."""
    f = frame.frame.payload.forward
    N = f.token_ids.len
    R = f.qo_indptr.len - 1
    cap = 3 * N + 2 * R + f.sampling_indices.len + 16
    i64 = np.zeros(max(N, 1), np.int64)
    i32 = np.zeros(cap, np.int32)
    err = C.create_string_buffer(512)
    n = lib().pie_hip_driver_plan(C.byref(f), page_size, total_pages, i64.ctypes.data,
                                  i32.ctypes.data, cap, err, len(err))
    if n < 0:
        raise ValueError(err.value.decode())
    tail = i32[n - 7:n]
    R2, N2, S = int(tail[0]), int(tail[1]), int(tail[2])
    o = 0
    out = {}
    for name, cnt in (("positions", N2), ("row_page_begin", N2), ("row_kv_len", N2),
                      ("seq_len", R2), ("sample_rows", S), ("sample_indptr", R2 + 1)):
        out[name] = i32[o:o + cnt].copy()
        o += cnt
    out["kv_slots"] = i64[:N2].copy()
    out.update(R=R2, N=N2, S=S, max_kv_len=int(tail[3]), pure_decode=bool(tail[4]),
               all_greedy=bool(tail[5]), has_user_masks=bool(tail[6]))
    return out
