"""Host session of the routed-expert MXFP8 FFN forward (binding of ``include/plk_mok.h``).

Plays the part of ``MoKHost`` in campaigns/mok/host/mok_port_host.py:72-289 for the forward
pass: owns the loaded pipeline image, fills a problem record from torch tensors, launches
on the current torch stream.  Tensors are only used as device memory.
"""
from __future__ import annotations

import ctypes
import json
from ctypes import byref, c_void_p, sizeof

import torch

from .backend import MokLinkInfo, MokProblem, PlkError, check, load_library

TILE_X = 128
MX_BLOCK = 32


def scale_pitch(k: int) -> int:
    """Bytes per row-major scale row: K/32 rounded up to a multiple of 16."""
    return ((k // MX_BLOCK) + 15) // 16 * 16


def scale_slots(k: int) -> int:
    """Number of 128-element ring slots along K (= dwords per row of a slot-major scale array)."""
    return (k + 127) // 128


def weight_scales_to_slot_major(sc: torch.Tensor, k: int) -> torch.Tensor:
    """Row-major weight scales [E, N, ld] -> the slot-major layout the GEMM reads, [E, K/128, N, 4]."""
    if not sc.is_cuda or not sc.is_contiguous() or sc.dim() != 3 or sc.dtype != torch.uint8:
        raise PlkError(3, "scales must be a contiguous 3-D uint8 device tensor")
    e, n, ld = sc.shape
    out = torch.empty((e, scale_slots(k), n, 4), dtype=torch.uint8, device=sc.device)
    lib = load_library()
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    for i in range(e):
        check(lib, lib.plk_mxfp8_scales_to_slot_major(sc[i].data_ptr(), n, k, ld, out[i].data_ptr(), stream))
    return out


def weight_codes_to_k64_tiled(q: torch.Tensor, k: int) -> torch.Tensor:
    """Row-major weight codes [E, N, ld] (ld >= k) -> the K-tiled layout the GEMM streams, [E, k/64, N, 64]."""
    if not q.is_cuda or not q.is_contiguous() or q.dim() != 3 or q.dtype != torch.uint8:
        raise PlkError(3, "codes must be a contiguous 3-D uint8 device tensor")
    e, n, ld = q.shape
    if k % 64 or ld < k:
        raise PlkError(3, "k must be a multiple of 64 and not exceed the row pitch")
    out = torch.empty((e, k // 64, n, 64), dtype=torch.uint8, device=q.device)
    lib = load_library()
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    for i in range(e):
        check(lib, lib.plk_mxfp8_codes_to_k64_tiled(q[i].data_ptr(), n, k, ld, out[i].data_ptr(), stream))
    return out


def link_info_from_json(link: dict) -> MokLinkInfo:
    """Translate a ``link.json`` (pipec link output) into the C record the session wants."""
    entries = {e["stage_id"]: e for e in link["params"]["entries"]}
    return MokLinkInfo(struct_bytes=sizeof(MokLinkInfo), params_bytes=link["params"]["total_bytes"],
                       framework_offset=entries["mok.framework"]["offset"], gemm_offset=entries["mok.gemm"]["offset"],
                       act_offset=entries["mok.act"]["offset"], threads=link["threads"],
                       dyn_lds_bytes=link["dyn_smem_bytes"], workgroups_per_cu=link.get("workgroups_per_cu", 1))


class MoKSession:
    def __init__(self, image: bytes, link: MokLinkInfo | dict | str):
        if isinstance(link, str):
            with open(link) as fh:
                link = json.load(fh)
        if isinstance(link, dict):
            link = link_info_from_json(link)
        self.lib = load_library()
        self.link = link
        handle = c_void_p()
        buf = ctypes.create_string_buffer(image, len(image))
        check(self.lib, self.lib.plk_mok_session_create(buf, len(image), byref(link), byref(handle)))
        self._handle = handle

    def close(self) -> None:
        if self._handle:
            check(self.lib, self.lib.plk_mok_session_destroy(self._handle))
            self._handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @staticmethod
    def problem(*, x_q, x_sc, row_token, tokens_per_expert, w_gate_q, w_gate_sc, w_up_q, w_up_sc, w_down_q, w_down_sc,
                hidden_q, hidden_sc, y, swiglu_limit: float = 7.0) -> MokProblem:
        """Build the problem record from CUDA tensors (shapes checked here, contents by the library).  The record
        keeps references to the tensors (``.tensors``), so it stays valid for as long as the caller holds it."""
        for name, t in dict(x_q=x_q, x_sc=x_sc, tokens_per_expert=tokens_per_expert, w_gate_q=w_gate_q,
                            w_gate_sc=w_gate_sc, w_up_q=w_up_q, w_up_sc=w_up_sc, w_down_q=w_down_q,
                            w_down_sc=w_down_sc, hidden_q=hidden_q, hidden_sc=hidden_sc, y=y).items():
            if not t.is_cuda or not t.is_contiguous():
                raise PlkError(3, f"{name} must be a contiguous device tensor")
        # activation code tensors may carry a padded last dimension (row pitch); the logical sizes come from
        # y [R, H] and the K-tiled weights [E, K/64, N, 64]
        t_rows, ldh = x_q.shape
        r, h = y.shape
        if w_gate_q.dim() != 4 or w_gate_q.shape[3] != 64:
            raise PlkError(3, "weight codes must be K-tiled [E, K/64, N, 64] (see weight_codes_to_k64_tiled)")
        e, _, i, _ = w_gate_q.shape
        ldi_q = hidden_q.shape[1]
        if h % 64 or i % 64 or tuple(w_gate_q.shape) != (e, h // 64, i, 64) or tuple(w_up_q.shape) != (e, h // 64, i, 64) or \
                tuple(w_down_q.shape) != (e, i // 64, h, 64):
            raise PlkError(3, "weight shapes disagree with y / each other")
        if hidden_q.shape[0] != r or y.dtype != torch.bfloat16 or ldh < h or ldi_q < i:
            raise PlkError(3, "hidden_q / y shapes disagree")
        ldsh, ldsi = scale_pitch(h), scale_pitch(i)
        if x_sc.shape[1] != ldsh or hidden_sc.shape[1] != ldsi:
            raise PlkError(3, "activation scale pitch must be K/32 rounded up to a multiple of 16")
        if tuple(w_gate_sc.shape) != (e, scale_slots(h), i, 4) or tuple(w_up_sc.shape) != (e, scale_slots(h), i, 4) or \
                tuple(w_down_sc.shape) != (e, scale_slots(i), h, 4):
            raise PlkError(3, "weight scales must be slot-major [E, K/128, N, 4] (see weight_scales_to_slot_major)")
        if tokens_per_expert.dtype != torch.int32 or (row_token is not None and row_token.dtype != torch.int32):
            raise PlkError(3, "tokens_per_expert and row_token must be int32")
        prob = MokProblem(struct_bytes=sizeof(MokProblem), num_tokens=t_rows, hidden=h, intermediate=i, num_experts=e,
                          routed_rows=r, ld_sc_h=ldsh, ld_sc_i=ldsi, ld_q_h=ldh, ld_q_i=ldi_q,
                          swiglu_limit=swiglu_limit,
                          x_q=x_q.data_ptr(), x_sc=x_sc.data_ptr(),
                          row_token=0 if row_token is None else row_token.data_ptr(),
                          tokens_per_expert=tokens_per_expert.data_ptr(),
                          w_gate_q=w_gate_q.data_ptr(), w_gate_sc=w_gate_sc.data_ptr(), w_up_q=w_up_q.data_ptr(),
                          w_up_sc=w_up_sc.data_ptr(), w_down_q=w_down_q.data_ptr(), w_down_sc=w_down_sc.data_ptr(),
                          hidden_q=hidden_q.data_ptr(), hidden_sc=hidden_sc.data_ptr(), y=y.data_ptr())
        # the record holds bare addresses: keep the tensors alive as long as it is (a caller may pass temporaries)
        prob.tensors = (x_q, x_sc, row_token, tokens_per_expert, w_gate_q, w_gate_sc, w_up_q, w_up_sc, w_down_q, w_down_sc,
                        hidden_q, hidden_sc, y)
        return prob

    def status(self, stream: int | None = None) -> int:
        """Waits for the stream, then returns and clears the launches' sticky status word (``plk_mok_status``): 0, or
        bit 0 = a dependency wait inside a one-launch forward gave up."""
        s = c_void_p(torch.cuda.current_stream().cuda_stream if stream is None else stream)
        word = ctypes.c_uint32(0)
        check(self.lib, self.lib.plk_mok_status(self._handle, s, byref(word)))
        return word.value

    def launches(self, n: int) -> None:
        """``plk_mok_session_launches``: 1 = one launch per forward whenever ``hidden_q`` allows it (the default), 2 = always
        gate/up then down as two launches (for a GPU that is shared with other work)."""
        check(self.lib, self.lib.plk_mok_session_launches(self._handle, n))

    def forward_static(self, problem: MokProblem, stream: int | None = None) -> None:
        """Both passes through the entry point that allocates nothing (``plk_mok_forward_static``): the params images
        go into a fixed area of device memory the library owns; calls that overlap on one GPU race on it."""
        s = c_void_p(torch.cuda.current_stream().cuda_stream if stream is None else stream)
        check(self.lib, self.lib.plk_mok_forward_static(self._handle, byref(problem), s))

    def forward(self, problem: MokProblem, stream: int | None = None, which: int = 0) -> None:
        """The whole forward (``which=0``: one launch when hidden_q's rows are whole 128-byte lines, else two) or one
        pass of it (1 = gate/up+SwiGLU+requant, 2 = down)."""
        s = c_void_p(torch.cuda.current_stream().cuda_stream if stream is None else stream)
        if which == 0:
            check(self.lib, self.lib.plk_mok_forward(self._handle, byref(problem), s))
        else:
            check(self.lib, self.lib.plk_mok_forward_pass(self._handle, byref(problem), which, s))


def code_pitch(k: int, align: int = 128) -> int:
    """Row pitch in bytes of an e4m3 operand whose rows start on `align`-byte boundaries."""
    return (k + align - 1) // align * align


def mxfp8_quantize_device(src: torch.Tensor, pitch: int | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantise a 2-D fp32 or bf16 device tensor along its last axis on the GPU.

    ``pitch`` pads every code row to that many bytes (pad bytes are zero)."""
    if not src.is_cuda or not src.is_contiguous() or src.dim() != 2 or src.dtype not in (torch.float32, torch.bfloat16):
        raise PlkError(3, "src must be a contiguous 2-D fp32/bf16 device tensor")
    rows, k = src.shape
    ld = scale_pitch(k)
    pitch = k if pitch is None else pitch
    q = torch.empty((rows, pitch), dtype=torch.uint8, device=src.device) if pitch == k else \
        torch.zeros((rows, pitch), dtype=torch.uint8, device=src.device)
    sc = torch.empty((rows, ld), dtype=torch.uint8, device=src.device)
    lib = load_library()
    check(lib, lib.plk_mxfp8_quantize(src.data_ptr(), int(src.dtype == torch.bfloat16), rows, k, q.data_ptr(), pitch,
                                      sc.data_ptr(), ld, c_void_p(torch.cuda.current_stream().cuda_stream)))
    return q, sc
