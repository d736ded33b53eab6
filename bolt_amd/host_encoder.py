"""Host-side driver of the int8 encoder layer: packs the weights once (load time) and runs
bolt_gfx950_encoder_layer_int8 on torch CUDA tensors. All arithmetic is in libbolt_gfx950.so."""
import ctypes as C

import numpy as np

from . import capi, host
from .capi import DF_TRANSPOSE, BoltEncoderLayerInt8, check, lib


class EncoderLayer:
    def __init__(self, torch, batch, seq, hidden, heads, ffn, P):
        """P: s8 weights [N, K] (wqkv, wo, w1, w2), fp32 per-channel scales (sqkv, so, s1, s2), fp32 biases
        (bqkv, bo, b1, b2, may be None) and LayerNorm parameters (ln1_g, ln1_b, ln2_g, ln2_b), numpy."""
        self.torch = torch
        dev = torch.device("cuda:0")
        self.keep = {}

        def put(a):
            return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)
        L = BoltEncoderLayerInt8()
        L.batch, L.seq, L.hidden, L.heads, L.ffn = batch, seq, hidden, heads, ffn
        for name, K, N in (("wqkv", hidden, 3 * hidden), ("wo", hidden, hidden), ("w1", hidden, ffn), ("w2", ffn, hidden)):
            blob, _, _ = host.mmm_transform_rhs(put(P[name]), DF_TRANSPOSE, K, N)      # [N, K] = transposed [K, N]
            self.keep[name] = blob
            setattr(L, name, blob.data_ptr())
        for name in ("sqkv", "so", "s1", "s2", "bqkv", "bo", "b1", "b2"):
            t = put(P.get(name))
            self.keep[name] = t
            setattr(L, name, C.cast(t.data_ptr() if t is not None else None, C.POINTER(C.c_float)))
        for cname, pname in (("ln1_gamma", "ln1_g"), ("ln1_beta", "ln1_b"), ("ln2_gamma", "ln2_g"), ("ln2_beta", "ln2_b")):
            t = put(P[pname])
            self.keep[cname] = t
            setattr(L, cname, C.cast(t.data_ptr(), C.POINTER(C.c_float)))
        self.L = L
        nbytes = C.c_size_t(0)
        check(lib().bolt_gfx950_encoder_layer_int8_workspace_bytes(C.byref(L), C.byref(nbytes)), "encoder_workspace_bytes")
        self.workspace = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
        self.tokens = batch * seq
        self.hidden = hidden

    def __call__(self, x, out=None):
        if out is None:
            out = self.torch.empty_like(x)
        check(lib().bolt_gfx950_encoder_layer_int8(C.byref(self.L), x.data_ptr(), out.data_ptr(), self.workspace.data_ptr(),
                                                  self.workspace.numel()), "encoder_layer")
        return out

    def intermediates(self):
        """fp32 intermediates the last call left in the workspace (views, not copies)."""
        offs = (C.c_size_t * 6)()
        check(lib().bolt_gfx950_encoder_layer_int8_workspace_layout(C.byref(self.L), offs), "encoder_workspace_layout")
        T, H, F = self.tokens, self.hidden, self.L.ffn
        shapes = (("qkv", 3 * H), ("ctx", H), ("attn_out", H), ("h1", H), ("ffn_pre", F), ("ffn_out", H))
        return {name: self.workspace[offs[i]:offs[i] + T * w * 4].view(self.torch.float32).view(T, w)
                for i, (name, w) in enumerate(shapes)}


class EncoderStack:
    """Several EncoderLayer objects run back to back by bolt_gfx950_encoder_stack_int8 (same batch, seq and hidden)."""

    def __init__(self, torch, layers):
        self.torch = torch
        self.layers = list(layers)   # keeps their weights alive
        n = len(self.layers)
        self.specs = (BoltEncoderLayerInt8 * n)(*[l.L for l in self.layers])
        nbytes = C.c_size_t(0)
        check(lib().bolt_gfx950_encoder_stack_int8_workspace_bytes(self.specs, n, C.byref(nbytes)), "encoder_stack_workspace_bytes")
        self.workspace = torch.empty(nbytes.value, dtype=torch.uint8, device=torch.device("cuda:0"))

    def __call__(self, x, out=None):
        if out is None:
            out = self.torch.empty_like(x)
        check(lib().bolt_gfx950_encoder_stack_int8(self.specs, len(self.layers), x.data_ptr(), out.data_ptr(),
                                                  self.workspace.data_ptr(), self.workspace.numel()), "encoder_stack")
        return out
