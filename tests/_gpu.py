"""GPU-side helpers for the parity tests: upload storage bits, run the C-ABI path through the
blitz_scale_amd.kernel mirror, bring results back as numpy."""
import numpy as np
import torch

from blitz_scale_amd import kernel as K
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_F32, BZ_ROPE_NONE

TORCH_OF = {BZ_F16: torch.float16, BZ_BF16: torch.bfloat16, BZ_E4M3: torch.uint8, BZ_F32: torch.float32}


def to_dev(bits, dtype):
    """numpy storage bits -> device tensor of the matching torch dtype."""
    if dtype == BZ_E4M3:
        return torch.from_numpy(np.ascontiguousarray(bits, np.uint8)).cuda()
    if dtype == BZ_F32:
        return torch.from_numpy(np.ascontiguousarray(bits, np.float32)).cuda()
    return torch.from_numpy(np.ascontiguousarray(bits, np.uint16).view(np.int16)).cuda().view(TORCH_OF[dtype])


def to_host_bits(t):
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def to_host_f32(t):
    return t.float().cpu().numpy()


class DeviceDecode:
    """Device image of a tests._util.DecodeProblem plus plan workspaces."""

    def __init__(self, p, float_ws_bytes=32 << 20, int_ws_bytes=8 << 20):
        self.p = p
        self.pool = to_dev(p.pool, p.kv_dtype)
        self.q = to_dev(p.q, p.dtype)
        self.pt = K.PageTable(p.B, p.P, p.Hkv, p.D, self.pool, layout=p.layout)
        self.pt.indices, self.pt.indptr, self.pt.last_page_len = p.indices, p.indptr, p.last_page_len
        self.pt.upload()
        self.float_ws = torch.empty(float_ws_bytes, dtype=torch.uint8, device="cuda")
        self.int_ws = torch.empty(int_ws_bytes, dtype=torch.uint8, device="cuda")
        self.handler = K.BlitzBatchDecodeHandler()
        self.k_scale = None if p.k_scale is None else torch.from_numpy(p.k_scale).cuda()
        self.v_scale = None if p.v_scale is None else torch.from_numpy(p.v_scale).cuda()

    def plan(self, split_tokens=0):
        p = self.p
        self.handler.plan(self.float_ws, self.float_ws.numel(), self.int_ws, self.int_ws.numel(), p.indptr,
                          p.last_page_len, p.B, p.Hq, p.Hkv, p.D, p.P, split_tokens=split_tokens)
        return self.handler.info()

    def decode(self, out_dtype=None, rope_mode=BZ_ROPE_NONE, rope_theta=1e4, sm_scale=0.0, want_lse=False, q=None):
        p = self.p
        out_dtype = p.dtype if out_dtype is None else out_dtype
        out = torch.full((p.B, p.Hq, p.D), float("nan"), dtype=TORCH_OF[out_dtype], device="cuda")
        lse = torch.empty((p.B, p.Hq), dtype=torch.float32, device="cuda") if want_lse else None
        K.batch_decode_attention(self.handler, self.q if q is None else q, self.pt, out, p.Hq, rope_mode=rope_mode,
                                 rope_theta=rope_theta, sm_scale=sm_scale, k_scale=self.k_scale,
                                 v_scale=self.v_scale, lse=lse)
        torch.cuda.synchronize()
        return (to_host_f32(out), lse.cpu().numpy()) if want_lse else to_host_f32(out)
