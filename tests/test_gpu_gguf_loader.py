"""GGUF file -> HBM: the loader puts a tensor's bytes on the device unchanged and the kernels run on
the handle it returns (load_quant_linear, crates/oxillama-arch/src/llama/model.rs:805-822)."""
import ctypes as C

import numpy as np
import pytest
import torch

import gguf_build as B
import oracle as O
from oxillama_amd import capi, gguf, synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def as_tensor(ptr, nbytes):
    """Copy nbytes from a raw device pointer to the host."""
    out = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    assert hip.hipMemcpy(out.data_ptr(), ptr, nbytes, 3) == 0  # device to device
    torch.cuda.synchronize()
    return out.cpu().numpy()


def model_file(tmp_path, big=False):
    n, k = (14336, 4096) if big else (96, 512)
    tensors, blobs, off = [], [], 0
    specs = [("blk.0.ffn_gate.weight", O.Q4_K, n, k), ("blk.0.ffn_down.weight", O.Q6_K, k // (4 if big else 1), n if big else 512),
             ("blk.0.attn_q.weight", O.Q8_0, 64, k), ("blk.0.attn_k.weight", O.Q5_K, 32, k)]
    for i, (name, t, rows, cols) in enumerate(specs):
        w = synth.weights(t, 50 + i, rows, cols) if t in O.ALL_TYPES else O.random_blocks(t, 50 + i, rows, cols)
        tensors.append((name, [rows, cols], t, off))
        blobs.append((off, w.tobytes()))
        off = B.align_up(off + w.size, 32)
    norm = synth.normal_f32(9, k)
    tensors.append(("blk.0.attn_norm.weight", [k], 0, off))
    blobs.append((off, norm.tobytes()))
    off += norm.nbytes
    tensors.append(("odd.weight", [3, 40], O.Q8_0, off))  # 40 columns: not whole blocks per row
    blobs.append((off, b"\0" * 136))
    off += 136
    tensors.append(("iq2.weight", [2, 256], 16, off))  # IQ2_XXS: parsed, but no kernel
    blobs.append((off, b"\0" * 132))
    off += 132
    data = bytearray(off)
    for o, b in blobs:
        data[o:o + len(b)] = b
    img = B.build(3, [("general.architecture", B.STRING, "llama"), ("llama.block_count", B.U32, 1)], tensors, bytes(data))
    p = tmp_path / "model.gguf"
    p.write_bytes(img)
    return p, specs, norm


@pytest.mark.parametrize("big", [False, True], ids=["small", "llama_shapes"])
def test_load_weights_and_run(hip, ref, tmp_path, big):
    path, specs, norm = model_file(tmp_path, big)
    g = gguf.GgufModel.load(path)
    assert g.architecture() == "llama" and g.n_tensors == len(specs) + 3
    for name, t, rows, cols in specs:
        print("load", name, flush=True)
        host_bytes = g.tensor_data(name)
        w = g.load_quant_linear(name)
        assert (w.tensor_type, w.shape, w.nbytes) == (t, [rows, cols], host_bytes.size)
        assert np.array_equal(as_tensor(w.device_ptr(), w.nbytes), host_bytes), "bytes on the device differ from the file"
        # the kernels take the handle's pointer as any other resident weights
        x = synth.normal_f32(3, cols)
        acts = ref.quantize_q8_0(x)
        d_acts = torch.from_numpy(acts).to(DEV)
        d_out = torch.zeros(rows, dtype=torch.float32, device=DEV)
        lib = capi.load()
        st = lib.oxq_matvec_q8_fused_dev(t, w.device_ptr(), d_acts.data_ptr(), d_out.data_ptr(), rows, cols, 0,
                                         C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert st == 0
        torch.cuda.synchronize()
        want = ref.matvec_q8_fused_mt(t, host_bytes, acts, rows, cols, 8)
        got = d_out.cpu().numpy()
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
        w.release()
    # any tensor's raw bytes into a caller's buffer (RMSNorm weights are F32 in GGUF files)
    d_norm = torch.empty(norm.size, dtype=torch.float32, device=DEV)
    g.upload_tensor("blk.0.attn_norm.weight", d_norm)
    assert np.array_equal(d_norm.cpu().numpy(), norm)
    with pytest.raises(hip.BufferTooSmall):
        g.upload_tensor("blk.0.attn_norm.weight", d_norm[:8])
    # what the loader refuses
    with pytest.raises(gguf.TensorNotFound):
        g.load_quant_linear("blk.7.attn_q.weight")
    with pytest.raises(hip.UnsupportedShape):
        g.load_quant_linear("odd.weight")
    with pytest.raises(hip.UnsupportedType):
        g.load_quant_linear("blk.0.attn_norm.weight")  # F32: no quantized kernel (and one-dimensional)
    with pytest.raises(hip.UnsupportedType):
        g.load_quant_linear("iq2.weight")
    g.close()


def test_truncated_file_is_reported_not_read(hip, tmp_path):
    path, specs, _ = model_file(tmp_path)
    img = path.read_bytes()
    cut = tmp_path / "cut.gguf"
    cut.write_bytes(img[:len(img) - 40000])
    g = gguf.GgufModel.load(cut)
    with pytest.raises(gguf.UnexpectedEof):
        g.load_quant_linear("blk.0.attn_k.weight")
    g.close()
