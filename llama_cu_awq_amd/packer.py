"""Repacking of AWQ checkpoints into the reference's .bin layout (what the reference's weight_packer.cpp does).

Old-format AWQ tensors (weight_packer.cpp:94-144, `OldAwqFormat = 1`):
  qweight int32 [K][N/8]  nibble i of a dword is column x + order_map[i], order_map = {0,2,4,6,1,3,5,7}
  qzeros  int32 [G][N/8]  same interleave, G = ceil(K/128)
  scales  fp16  [G][N]
become, one row per output column n:
  weight u32 [N][K/8]  element k in bits 4*(k%8);  zeros u32 [N][ceil(G/8)];  scales fp16 [N][G].
Padding nibbles of the last zeros dword are written as 0 here (the reference's tool leaves whatever lay beyond its
temporary buffer there, weight_packer.cpp:117-121; the kernels never read them).
"""
import numpy as np

from . import synth

ORDER_MAP = np.array([0, 2, 4, 6, 1, 3, 5, 7])


def deinterleave(packed):
    """int32/uint32 [rows][cols/8] in AWQ order -> uint8 [rows][cols] (weight_packer.cpp:96-107)."""
    packed = np.ascontiguousarray(packed).view(np.uint32)
    rows, c8 = packed.shape
    out = np.empty((rows, c8, 8), dtype=np.uint8)
    for i in range(8):
        out[:, :, ORDER_MAP[i]] = (packed >> np.uint32(4 * i)) & np.uint32(0xF)
    return out.reshape(rows, c8 * 8)


def interleave(vals):
    """Inverse of deinterleave: uint8 [rows][cols] -> uint32 [rows][cols/8] in AWQ order."""
    rows, cols = vals.shape
    v = vals.reshape(rows, cols // 8, 8).astype(np.uint32)
    out = np.zeros((rows, cols // 8), dtype=np.uint32)
    for i in range(8):
        out |= v[:, :, ORDER_MAP[i]] << np.uint32(4 * i)
    return out


def repack_old_awq(qweight, qzeros, scales, K, N):
    """Old-format AWQ (qweight [K][N/8], qzeros [G][N/8], scales [G][N]) -> (weight, zeros, scales) of the .bin layout."""
    pwh, pzh, sh = synth.strides(K)
    q = deinterleave(qweight)[:K, :N]   # [K][N]
    z = deinterleave(qzeros)[:sh, :N]   # [G][N]
    weight = synth.pack_nibbles(np.ascontiguousarray(q.T), pwh)
    zeros = synth.pack_nibbles(np.ascontiguousarray(z.T), pzh)
    sc = np.ascontiguousarray(np.asarray(scales).view(np.float16).reshape(sh, N).T)
    return weight, zeros, sc


def write_model(path_or_none, cfg, tensors):
    """Assemble a .bin image (llama2_q4.cu:220-246 / weight_packer.cpp:256-292 order).

    tensors: dict with 'embed', 'lm_head', 'norm' (fp16 arrays) and per layer l the keys
    f'{l}.{name}' for name in q_proj,k_proj,v_proj,o_proj,up_proj,gate_proj,down_proj -> (weight, zeros, scales)
    and f'{l}.input_layernorm', f'{l}.post_attention_layernorm' (fp16).
    """
    parts = [np.array([cfg[k] for k in ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len")], dtype=np.int32).view(np.uint8),
             np.array([cfg.get("rope_theta", 10000.0)], dtype=np.float32).view(np.uint8)]

    def put(a):
        parts.append(np.ascontiguousarray(a).reshape(-1).view(np.uint8))

    put(tensors["embed"])
    put(tensors["lm_head"])
    put(tensors["norm"])
    for l in range(cfg["n_layers"]):
        for name in ("q_proj", "k_proj", "v_proj", "o_proj", "up_proj", "gate_proj", "down_proj"):
            w, z, s = tensors[f"{l}.{name}"]
            put(w)
            put(z)
            put(s)
        put(tensors[f"{l}.input_layernorm"])
        put(tensors[f"{l}.post_attention_layernorm"])
    img = np.concatenate(parts)
    if path_or_none:
        img.tofile(path_or_none)
    return img
