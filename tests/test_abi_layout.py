"""Layout of include/pie_driver_abi.h against the reference boundary header (CPU only).

Both headers define the same struct names, so each is compiled into its own small program
that prints sizeof / offsetof for every descriptor field; the outputs must be identical.
The reference header is only read when the reference tree is present (this container);
elsewhere the test checks our header against ctypes' independent layout computation."""
import ctypes as C
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
REF = Path("/root/reference/driver/bridge/include/pie_bridge.h")

# (struct, [fields]); a slice field `f` is `f.ptr`/`f.len` here and `f_ptr`/`f_len` there
STRUCTS = {
    "PieAdapterBindingDesc": ["adapter_id", "seed"],
    "PieBrleDesc": ["@buffer", "total_size"],
    "PieSamplerDesc": ["kind", "temperature", "seed", "k", "p", "num_tokens", "token_id", "@token_ids"],
    "PieForwardRequestDesc": [
        "@token_ids", "@position_ids", "@kv_page_indices", "@kv_page_indptr", "@kv_last_page_lens",
        "@qo_indptr", "@rs_slot_ids", "@rs_slot_flags", "@masks", "@mask_indptr", "@logit_masks",
        "@logit_mask_indptr", "@sampling_indices", "@sampling_indptr", "@samplers",
        "@sampler_indptr", "@adapter_bindings", "@spec_token_ids", "@spec_position_ids",
        "@spec_indptr", "@output_spec_flags", "@context_ids", "single_token_mode", "has_user_mask",
        "@image_indptr", "@image_grids", "@image_anchor_positions", "@image_pixels",
        "@image_pixel_indptr", "@image_mrope_positions", "@image_mrope_indptr",
        "@image_patch_positions", "@image_anchor_rows", "@audio_features", "@audio_feature_indptr",
        "@audio_anchor_rows", "@audio_indptr"],
    "PieForwardResponseDesc": [
        "num_requests", "@tokens_indptr", "@tokens", "@dists_req_indptr", "@dists_kv_indptr",
        "@dists_ids", "@dists_probs", "@logits_req_indptr", "@logits_byte_indptr", "@logits_bytes",
        "@logprobs_req_indptr", "@logprobs_val_indptr", "@logprobs_values", "@entropies_indptr",
        "@entropies", "@spec_indptr", "@spec_tokens", "@spec_positions", "probe_wire_parse_us",
        "probe_plan_us", "probe_h2d_us", "probe_kernel_launch_us", "probe_sync_us",
        "probe_response_build_us"],
    "PieCopyRequestDesc": ["dir", "@srcs", "@dsts", "resource"],
    "PieAdapterRequestDesc": ["op", "adapter_id", "@path"],
    "PieStatusResponseDesc": ["status"],
    "PieRequestPayloadDesc": ["kind", "forward", "copy", "adapter"],
    "PieResponsePayloadDesc": ["kind", "forward", "status"],
    "PieFrameDesc": ["driver_id", "payload"],
    "PieResponseFrameDesc": ["driver_id", "aborted", "payload"],
    "PieInProcVTable": ["recv", "send_response", "ctx"],
}


def dump_program(header: Path, ours: bool) -> str:
    lines = ["#include <cstddef>", "#include <cstdio>", f'#include "{header}"', "int main() {"]
    for st, fields in STRUCTS.items():
        lines.append(f'  std::printf("{st} %zu\\n", sizeof({st}));')
        for f in fields:
            if f.startswith("@"):
                n = f[1:]
                p, l = (f"{n}.ptr", f"{n}.len") if ours else (f"{n}_ptr", f"{n}_len")
                lines.append(f'  std::printf("{st}.{n}.ptr %zu\\n", offsetof({st}, {p}));')
                lines.append(f'  std::printf("{st}.{n}.len %zu\\n", offsetof({st}, {l}));')
            else:
                lines.append(f'  std::printf("{st}.{f} %zu\\n", offsetof({st}, {f}));')
    lines += ["  return 0;", "}"]
    return "\n".join(lines)


def run_dump(tmp_path, header, ours):
    src = tmp_path / ("ours.cpp" if ours else "ref.cpp")
    exe = tmp_path / ("ours" if ours else "ref")
    src.write_text(dump_program(header, ours))
    subprocess.run(["g++", "-std=c++17", "-Wno-invalid-offsetof", "-o", str(exe), str(src)], check=True)
    return subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout


def test_layout_matches_reference_header(tmp_path):
    if not REF.exists():
        pytest.skip("reference tree not present")
    ours = run_dump(tmp_path, ROOT / "include" / "pie_driver_abi.h", True)
    ref = run_dump(tmp_path, REF, False)
    assert ours == ref
    assert "PieFrameDesc" in ours and len(ours.splitlines()) > 150


def test_ctypes_mirror_matches_header(tmp_path):
    from pie_amd import driver as drv

    ours = dict(l.split() for l in run_dump(tmp_path, ROOT / "include" / "pie_driver_abi.h", True).splitlines())
    pairs = {"PieForwardRequestDesc": drv.ForwardRequestDesc, "PieForwardResponseDesc": drv.ForwardResponseDesc,
             "PieFrameDesc": drv.FrameDesc, "PieResponseFrameDesc": drv.ResponseFrameDesc,
             "PieSamplerDesc": drv.SamplerDesc, "PieBrleDesc": drv.BrleDesc,
             "PieCopyRequestDesc": drv.CopyRequestDesc, "PieAdapterRequestDesc": drv.AdapterRequestDesc,
             "PieRequestPayloadDesc": drv.RequestPayloadDesc, "PieResponsePayloadDesc": drv.ResponsePayloadDesc,
             "PieInProcVTable": drv.InProcVTable}
    for name, ct in pairs.items():
        assert C.sizeof(ct) == int(ours[name]), name
        for fname, _ in ct._fields_:
            off = getattr(ct, fname).offset
            key = f"{name}.{fname}" if f"{name}.{fname}" in ours else f"{name}.{fname}.ptr"
            assert off == int(ours[key]), key


def test_driver_library_exports_declared_symbols():
    from test_abi_exports import declared

    lib = C.CDLL(str(ROOT / "pie_amd" / "libpie_driver_hip.so"))
    names = declared(ROOT / "include" / "pie_driver_abi.h", "pie_")
    assert "pie_driver_hip_run_inproc" in names and "pie_driver_hip_request_stop" in names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
