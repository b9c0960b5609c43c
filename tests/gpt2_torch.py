"""A textbook GPT-2 forward written with torch library routines only (float64 on the
CPU). Used to pin the oracle's whole-model wiring: it shares no code with it."""
import torch
import torch.nn.functional as F


def forward(params, tensors, tokens, dtype=torch.float64):
    """Returns (logits of the last token, {tap name: [T,d] tensor})."""
    L, H, d = params["n_layer"], params["n_head"], params["n_embd"]
    hs = d // H
    t = lambda name: torch.from_numpy(tensors[name]).to(dtype)
    idx = torch.as_tensor(tokens, dtype=torch.long)
    T = idx.shape[0]
    taps = {}
    x = t("transformer.wte.weight")[idx] + t("transformer.wpe.weight")[:T]
    taps["tok_pos_emb"] = x
    for i in range(L):
        p = f"transformer.h.{i}."
        h = F.layer_norm(x, (d,), t(p + "ln_1.weight"), t(p + "ln_1.bias"), eps=1e-5)
        taps[f"block{i}_ln1"] = h
        qkv = h @ t(p + "attn.c_attn.weight") + t(p + "attn.c_attn.bias")       # HF Conv1D: weight is [in, out]
        q, k, v = qkv.split(d, dim=1)
        heads = lambda a: a.reshape(T, H, hs).transpose(0, 1)
        o = F.scaled_dot_product_attention(heads(q), heads(k), heads(v), is_causal=True)
        a = o.transpose(0, 1).reshape(T, d) @ t(p + "attn.c_proj.weight") + t(p + "attn.c_proj.bias")
        taps[f"block{i}_attn"] = a
        x = x + a
        taps[f"block{i}_r1"] = x
        h = F.layer_norm(x, (d,), t(p + "ln_2.weight"), t(p + "ln_2.bias"), eps=1e-5)
        taps[f"block{i}_ln2"] = h
        m = F.gelu(h @ t(p + "mlp.c_fc.weight") + t(p + "mlp.c_fc.bias"), approximate="tanh")
        m = m @ t(p + "mlp.c_proj.weight") + t(p + "mlp.c_proj.bias")
        taps[f"block{i}_mlp"] = m
        x = x + m
        taps[f"block{i}_r2"] = x
        taps[f"kv{i}_k"], taps[f"kv{i}_v"] = k, v
    h = F.layer_norm(x, (d,), t("transformer.ln_f.weight"), t("transformer.ln_f.bias"), eps=1e-5)
    taps["ln_f"] = h
    logits = h[-1] @ t("transformer.wte.weight").T
    return logits, taps
