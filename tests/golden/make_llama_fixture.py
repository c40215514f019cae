"""Writes a small Llama-family model directory in the on-disk format the reference's convert tools
produce and its loader reads (config.ini keys: src/models/common_decoder.h:176-233; file names and
shapes: src/layers/decoder_block.h:205-343, common_decoder.h:857-874, llama.cpp:46-51):

    config.ini                                  one [llama] section
    model.wte.bin                               [vocab, hidden]
    model.layers.N.attention.query_key_value.weight.0.bin   [hidden, (q + 2 kv) * head]
    model.layers.N.attention.dense.weight.0.bin             [q * head, hidden]
    model.layers.N.mlp.{gate_proj,up_proj}.weight.0.bin     [hidden, inter]
    model.layers.N.mlp.down_proj.weight.0.bin               [inter, hidden]
    model.layers.N.{input,post_attention}_layernorm.weight.bin  [hidden]
    model.final_layernorm.weight.bin            [hidden]
    model.lm_head.weight.bin                    [vocab, hidden]
  a Mixtral directory (`experts=8`; section [mixtral], src/xfastertransformer/tools/mixtral_convert.py:120-160,
  src/layers/decoder_block.h:640-676) holds instead of the three mlp matrices
    model.layers.N.moe.gate.weight.bin                      [hidden, experts]   (the router)
    model.layers.N.moe.sparse_experts.E.w1.0.bin            [hidden, inter]     (gate)
    model.layers.N.moe.sparse_experts.E.w2.0.bin            [hidden, inter]     (up)
    model.layers.N.moe.sparse_experts.E.w3.0.bin            [inter, hidden]     (down)
  pre-quantised directories hold .qweight.0.bin (int8, or two 4-bit codes per byte with the even
  column in the low nibble) + .scales.0.bin + .zeros.0.bin (fp32 per output column) instead of
  .weight.0.bin.

The weights are seeded random numbers (there is no checkpoint to convert here); the function
returns them exactly as the files hold them, so a test can build the same model directly.

    python tests/golden/make_llama_fixture.py OUT_DIR [--weight-type fp32|fp16|bf16] [--quant int8|uint4]
"""
import argparse
import os

import numpy as np

TINY = dict(layers=2, hidden=256, inter=512, heads=2, kv_heads=1, head=128, vocab=512, max_pos=256, eps=1e-5,
            rope_theta=10000.0)


def _bf16_round(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def _store(path, a, weight_type):
    """Writes `a` in the file's element type and returns the values the file now holds (fp32)."""
    a = np.ascontiguousarray(a, np.float32)
    if weight_type == "fp32":
        a.tofile(path)
        return a
    if weight_type == "fp16":
        h = a.astype(np.float16)
        h.tofile(path)
        return h.astype(np.float32)
    if weight_type == "bf16":
        b = _bf16_round(a)
        b.tofile(path)
        return (b.astype(np.uint32) << 16).view(np.float32).reshape(a.shape)
    raise ValueError(weight_type)


def _quantize(w, quant):
    """Per-output-column asymmetric codes: w ~ scale * q + zero."""
    lo, hi = w.min(axis=0), w.max(axis=0)
    if quant == "int8":
        scale = np.maximum((hi - lo) / 255.0, 1e-8).astype(np.float32)
        zero = (lo + 128.0 * scale).astype(np.float32)
        q = np.clip(np.rint((w - zero) / scale), -128, 127).astype(np.int8)
        return q, scale, zero
    scale = np.maximum((hi - lo) / 15.0, 1e-8).astype(np.float32)
    zero = lo.astype(np.float32)
    q = np.clip(np.rint((w - zero) / scale), 0, 15).astype(np.uint8)
    return q, scale, zero


def write_model_dir(out, cfg=None, seed=0, weight_type="fp32", quant=None, experts=0):
    cfg = dict(TINY if cfg is None else cfg)
    assert not (experts and quant), "pre-quantised Mixtral directories are not written here"
    os.makedirs(out, exist_ok=True)
    L, H, I, qh, kvh, D, V = (cfg[k] for k in ("layers", "hidden", "inter", "heads", "kv_heads", "head", "vocab"))
    with open(os.path.join(out, "config.ini"), "w") as f:
        f.write("[mixtral]\n" if experts else "[llama]\n")
        f.write("model_name = fixture\n")
        f.write(f"head_num = {qh}\nkv_head_num = {kvh}\nsize_per_head = {D}\ninter_size = {I}\n")
        f.write(f"max_pos_seq_len = {cfg['max_pos']}\nnum_layer = {L}\nlayernorm_eps = {cfg['eps']}\n")
        f.write("layernorm_type = pre_layernorm\nactivation_type = silu\n")
        f.write(f"rope_theta = {cfg['rope_theta']}\nhas_post_decoder_layernorm = 1\nvocab_size = {V}\n")
        f.write("start_id = 1\nend_id = 2\n")
        f.write(f"weight_data_type = {weight_type}\n")
        if experts:
            f.write("attn_params_type = GQAttnParams\nffn_params_type = MixtralFFNParams\n")
            if experts != 8:
                f.write(f"sparse_experts = {experts}\n")
        if quant:
            f.write(f"quant_qweight_data_type = {quant}\nquant_scales_data_type = fp32\nquant_zeros_data_type = fp32\n")
            f.write("quant_groupsize = -1\n")
    rng = np.random.default_rng(seed)
    held = {"cfg": cfg, "layers": []}

    def matrix(l, stem, K, N, std):
        w = (rng.standard_normal((K, N)) * std).astype(np.float32)
        base = os.path.join(out, f"model.layers.{l}.{stem}")
        if not quant:
            return {"w": _store(base + ".weight.0.bin", w, weight_type)}
        q, scale, zero = _quantize(w, quant)
        if quant == "int8":
            q.tofile(base + ".qweight.0.bin")
        else:
            (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8).tofile(base + ".qweight.0.bin")
        scale.tofile(base + ".scales.0.bin")
        zero.tofile(base + ".zeros.0.bin")
        return {"q": q, "scale": scale, "zero": zero, "w": (scale.astype(np.float64) * q + zero).astype(np.float32)}  # one rounding, as fmaf(scale, q, zero)

    for l in range(L):
        lay = {}
        lay["qkv"] = matrix(l, "attention.query_key_value", H, (qh + 2 * kvh) * D, 0.05)
        lay["o"] = matrix(l, "attention.dense", qh * D, H, 0.05)
        if experts:
            lay["router"] = _store(os.path.join(out, f"model.layers.{l}.moe.gate.weight.bin"),
                                   rng.standard_normal((H, experts)) * 0.2, weight_type)
            lay["experts"] = []
            for e in range(experts):
                base = os.path.join(out, f"model.layers.{l}.moe.sparse_experts.{e}.")
                lay["experts"].append({"gate": _store(base + "w1.0.bin", rng.standard_normal((H, I)) * 0.05, weight_type),
                                       "up": _store(base + "w2.0.bin", rng.standard_normal((H, I)) * 0.05, weight_type),
                                       "down": _store(base + "w3.0.bin", rng.standard_normal((I, H)) * 0.05, weight_type)})
        else:
            lay["gate"] = matrix(l, "mlp.gate_proj", H, I, 0.05)
            lay["up"] = matrix(l, "mlp.up_proj", H, I, 0.05)
            lay["down"] = matrix(l, "mlp.down_proj", I, H, 0.05)
        lay["ln1"] = _store(os.path.join(out, f"model.layers.{l}.input_layernorm.weight.bin"),
                            1.0 + 0.1 * rng.standard_normal(H), weight_type)
        lay["ln2"] = _store(os.path.join(out, f"model.layers.{l}.post_attention_layernorm.weight.bin"),
                            1.0 + 0.1 * rng.standard_normal(H), weight_type)
        held["layers"].append(lay)
    held["wte"] = _store(os.path.join(out, "model.wte.bin"), rng.standard_normal((V, H)), weight_type)
    held["final_norm"] = _store(os.path.join(out, "model.final_layernorm.weight.bin"), 1.0 + 0.1 * rng.standard_normal(H),
                                weight_type)
    held["lm_head"] = _store(os.path.join(out, "model.lm_head.weight.bin"), rng.standard_normal((V, H)) * 0.1, weight_type)
    return held


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("out")
    ap.add_argument("--weight-type", default="fp32", choices=["fp32", "fp16", "bf16"])
    ap.add_argument("--quant", default=None, choices=["int8", "uint4"])
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--experts", type=int, default=0, help="8: a Mixtral directory")
    a = ap.parse_args()
    write_model_dir(a.out, None, a.seed, a.weight_type, a.quant, a.experts)
    print("wrote", a.out)
