"""One local-encoder forward (csrc/models/local_encoder.c:193-281) through each implementation the
tests compare: the CPU restatement, the reference build on host tensors, the library's entry point
and the reference's own caller code on device tensors.  Not collected by pytest."""
import ctypes as C

import numpy as np

from fblt_amd import abi, decoder, encoder
from oracle import binding

PRIME = 1000003
POOLS = {"mean": abi.BLT_POOL_MEAN, "max": abi.BLT_POOL_MAX}


def rope_tables(orc, c):
    hd = c["E"] // c["H"]
    cos, sin = (np.empty(c["T"] * (hd // 2), dtype=np.float32) for _ in range(2))
    assert orc.orc_rope_precompute(c["T"], 500000.0, hd, binding.fptr(cos), binding.fptr(sin)) == 0
    return cos.reshape(c["T"], hd // 2), sin.reshape(c["T"], hd // 2)


def bound(orc, c, weights, backend, place):
    cos, sin = rope_tables(orc, c)
    return encoder.bind(weights, cos, sin, backend, place, c["E"], c["H"], c["XH"], c["hidden"], c["T"], c["ngrams"],
                        c["vocab"], PRIME, normalize=c["normalize"], patch_dim=c["E"] * c["k"] if c["k"] > 1 else 0,
                        window=c["window"], all_layers=c["all_layers"], placement=c["placement"],
                        pool=POOLS[c["pool"]])


def docs_arg(c):
    """(array or None, num_docs) in the mask builder's convention (entry d starts document d + 1)."""
    if not c["docs"]:
        return None, 0
    return abi.size_array(c["docs"]), len(c["docs"]) + 1


def outputs(c, lengths):
    P = len(lengths)
    return np.zeros((P, c["E"] * c["k"]), dtype=np.float32), np.zeros((c["T"], c["E"]), dtype=np.float32)


def run_oracle(orc, c, data, lengths, weights):
    enc = bound(orc, c, weights, abi.BLT_BACKEND_CPU, decoder.host_place)
    patches = decoder.patch_table(lengths)
    docs, num_docs = docs_arg(c)
    p_out, h_out = outputs(c, lengths)
    rc = orc.orc_local_encoder_forward(enc.ptr, data.ctypes.data_as(C.POINTER(C.c_uint8)), c["T"], patches,
                                       len(lengths), docs, num_docs, binding.fptr(p_out.reshape(-1)),
                                       binding.fptr(h_out.reshape(-1)))
    assert rc == 0, rc
    return p_out, h_out


def run_reference(ref, orc, c, data, lengths, weights):
    """blt_local_encoder_forward of the reference build, host tensors."""
    CPU = abi.BLT_BACKEND_CPU
    enc = bound(orc, c, weights, CPU, decoder.host_place)
    patches = decoder.patch_table(lengths)
    docs, num_docs = docs_arg(c)
    p_out, h_out = outputs(c, lengths)
    tb = abi.tensor_view(data.ctypes.data, data.shape, CPU, dtype=abi.BLT_DTYPE_UINT8)
    tp, th = abi.tensor_view(p_out.ctypes.data, p_out.shape, CPU), abi.tensor_view(h_out.ctypes.data, h_out.shape, CPU)
    arena = ref.blt_arena_create(256 << 20, CPU)
    try:
        ref.blt_local_encoder_forward(enc.ptr, C.byref(tb), patches, len(lengths), docs, num_docs, C.byref(tp),
                                      C.byref(th), arena)
    finally:
        ref.blt_arena_destroy(arena)
    return p_out, h_out


def run_device(entry, lib, orc, c, data, lengths, weights, bytes_on_device=True):
    """`entry` = a blt_local_encoder_forward with the reference's signature, on device tensors."""
    import torch
    HIP = abi.BLT_BACKEND_HIP
    enc = bound(orc, c, weights, HIP, decoder.device_place)
    patches = decoder.patch_table(lengths)
    docs, num_docs = docs_arg(c)
    P = len(lengths)
    p_out = torch.zeros((P, c["E"] * c["k"]), dtype=torch.float32, device="cuda")
    h_out = torch.zeros((c["T"], c["E"]), dtype=torch.float32, device="cuda")
    if bytes_on_device:
        tbytes = torch.from_numpy(data).cuda()
        tb = abi.tensor_view(tbytes.data_ptr(), data.shape, HIP, dtype=abi.BLT_DTYPE_UINT8)
    else:
        tb = abi.tensor_view(data.ctypes.data, data.shape, abi.BLT_BACKEND_CPU, dtype=abi.BLT_DTYPE_UINT8)
    tp = abi.tensor_view(p_out.data_ptr(), tuple(p_out.shape), HIP)
    th = abi.tensor_view(h_out.data_ptr(), tuple(h_out.shape), HIP)
    arena = lib.blt_arena_create(256 << 20, HIP)
    try:
        entry(enc.ptr, C.byref(tb), patches, P, docs, num_docs, C.byref(tp), C.byref(th), arena)
        lib.blt_backend_pass_sync_hip()
        return p_out.cpu().numpy(), h_out.cpu().numpy()
    finally:
        lib.blt_arena_destroy(arena)
