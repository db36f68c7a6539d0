"""Synthetic random-init models in the reference's on-disk formats.

Everything here is host-side numpy: random quantized super-blocks in the exact GGUF byte layouts
(quantization.h:57-124), a model builder for the BASELINE.json shapes with the "Q4_K_M" tensor-type
mix, and a GGUF-v3 writer (gguf_parser.cpp:134-528 is the reader it targets).

Scales are chosen so that dequantized weights have std ~= gain/sqrt(fan_in): activations stay O(1)
through any depth, logits are finite and the greedy top-2 gap is far above the fp32 tolerance.
"""
import struct

import numpy as np

F32, Q8_0, Q4_K, Q6_K, Q8_K = 0, 8, 12, 14, 15
BF16 = 30  # accepted by tl_model_set_tensor (widened to F32 at upload); a uint16 array
BLOCK_BYTES = {F32: 4, Q8_0: 34, Q4_K: 144, Q6_K: 210, Q8_K: 290, BF16: 2}
BLOCK_ELEMS = {F32: 1, Q8_0: 32, Q4_K: 256, Q6_K: 256, Q8_K: 256, BF16: 1}
TYPE_NAMES = {F32: "F32", Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K", Q8_K: "Q8_K"}


def tensor_bytes(typ, rows, cols):
    return rows * cols // BLOCK_ELEMS[typ] * BLOCK_BYTES[typ]


def _put_f16(blocks, off, vals):
    blocks[:, off:off + 2] = np.asarray(vals, np.float16).reshape(-1, 1).view(np.uint8)


def random_blocks(typ, nblocks, rng, w_std=0.02):
    """`nblocks` random blocks of `typ` as a uint8 array [nblocks, block_bytes]; payload bytes are
    uniform random, fp16 super-scales are drawn so the dequantized weights have std ~= w_std."""
    bb = BLOCK_BYTES[typ]
    b = rng.integers(0, 256, size=(nblocks, bb), dtype=np.uint8)
    u = rng.uniform(0.6, 1.4, size=nblocks)
    if typ == Q4_K:
        # w = d*sc*q - dmin*m, sc,m in [0,63], q in [0,15]: std(w) ~= d * 36.4 * 4.6 when centred
        d = w_std / 167.0 * u
        _put_f16(b, 0, d)
        _put_f16(b, 2, d * rng.uniform(6.5, 8.5, size=nblocks))  # ~zero-mean weights
    elif typ == Q6_K:
        # w = d*sc*q, sc int8 (kept in [-32,31]), q in [-32,31]: std ~= d * 18.5 * 18.5
        sc = rng.integers(-32, 32, size=(nblocks, 16), dtype=np.int8)
        b[:, 192:208] = sc.view(np.uint8)
        _put_f16(b, 208, w_std / 342.0 * u)
    elif typ in (Q8_0, Q8_K):
        # w = d*q, q int8 uniform: std ~= d * 73.9
        _put_f16(b, 0, w_std / 73.9 * u)
    else:
        raise ValueError(typ)
    return b


EDGE_F16 = [0x0000, 0x8000, 0x0001, 0x8001, 0x03ff, 0x83ff, 0x0400, 0x3c00, 0xbc00, 0x7bff, 0xfbff,
            0x1a3c, 0x9a3c, 0x2e66]
"""fp16 scale edge cases: +-0, smallest/largest subnormal, smallest normal, +-1, +-max finite, a few
ordinary values incl. negatives (Q8 scales take |d|, quantization.cpp:85-87)."""


def edge_blocks(typ, rng):
    """Blocks whose fp16 scale fields walk EDGE_F16 (both d and dmin for Q4_K), random payload."""
    n = len(EDGE_F16)
    b = rng.integers(0, 256, size=(n, BLOCK_BYTES[typ]), dtype=np.uint8)
    e = np.array(EDGE_F16, np.uint16)
    off = 208 if typ == Q6_K else 0
    b[:, off:off + 2] = e.reshape(-1, 1).view(np.uint8)
    if typ == Q4_K:
        b[:, 2:4] = np.roll(e, 3).reshape(-1, 1).view(np.uint8)
    return b


# ---- model shapes -----------------------------------------------------------------
SHAPES = {
    "tiny": dict(hidden=256, inter=512, n_heads=4, n_kv_heads=2, n_layers=3, vocab=64, max_pos=128,
                 eps=1e-5, rope_theta=10000.0),
    "tiny-gqa": dict(hidden=512, inter=1024, n_heads=8, n_kv_heads=2, n_layers=2, vocab=512, max_pos=256,
                     eps=1e-5, rope_theta=10000.0),
    "tiny-tp": dict(hidden=1024, inter=2048, n_heads=16, n_kv_heads=4, n_layers=2, vocab=512, max_pos=128,
                    eps=1e-5, rope_theta=10000.0),
    "tinyllama-1.1b": dict(hidden=2048, inter=5632, n_heads=32, n_kv_heads=4, n_layers=22, vocab=32000,
                           max_pos=2048, eps=1e-5, rope_theta=10000.0),
    "llama-3.2-3b": dict(hidden=3072, inter=8192, n_heads=24, n_kv_heads=8, n_layers=28, vocab=128256,
                         max_pos=2048, eps=1e-5, rope_theta=500000.0),
    "llama-3-8b": dict(hidden=4096, inter=14336, n_heads=32, n_kv_heads=8, n_layers=32, vocab=128256,
                       max_pos=8192, eps=1e-5, rope_theta=500000.0),
    "llama-3-70b": dict(hidden=8192, inter=28672, n_heads=64, n_kv_heads=8, n_layers=80, vocab=128256,
                        max_pos=8192, eps=1e-5, rope_theta=500000.0),
}


def tensor_plan(cfg, mix="q4_k_m"):
    """[(name, type, rows, cols)] in file order. mix: 'q4_k_m' (Q4_K except attn_v/ffn_down
    Q6_K on layers i<L/8 || i>=7L/8 || (i-L/8)%3==2, output Q6_K), 'q6_k', 'q8_0', 'q4_k'."""
    H, I, L, V = cfg["hidden"], cfg["inter"], cfg["n_layers"], cfg["vocab"]
    kvd = cfg["n_kv_heads"] * (H // cfg["n_heads"])
    base = {"q4_k_m": Q4_K, "q4_k": Q4_K, "q6_k": Q6_K, "q8_0": Q8_0}[mix]

    def more_bits(i):
        return mix == "q4_k_m" and (i < L // 8 or i >= 7 * L // 8 or (i - L // 8) % 3 == 2)

    plan = [("token_embd.weight", base, V, H)]
    for i in range(L):
        hi = Q6_K if more_bits(i) else base
        plan += [
            (f"blk.{i}.attn_norm.weight", F32, 1, H),
            (f"blk.{i}.attn_q.weight", base, H, H),
            (f"blk.{i}.attn_k.weight", base, kvd, H),
            (f"blk.{i}.attn_v.weight", hi, kvd, H),
            (f"blk.{i}.attn_output.weight", base, H, H),
            (f"blk.{i}.ffn_norm.weight", F32, 1, H),
            (f"blk.{i}.ffn_gate.weight", base, I, H),
            (f"blk.{i}.ffn_up.weight", base, I, H),
            (f"blk.{i}.ffn_down.weight", hi, H, I),
        ]
    plan += [("output_norm.weight", F32, 1, H),
             ("output.weight", Q6_K if mix == "q4_k_m" else base, V, H)]
    return plan


def weight_bytes_per_token(cfg, mix="q4_k_m"):
    """Algorithmic weight bytes one decoded token must read (SURVEY §8d B_tok without the KV terms):
    every projection + output.weight + ONE row of token_embd."""
    total = 0
    for name, typ, rows, cols in tensor_plan(cfg, mix):
        if typ == F32:
            continue
        total += tensor_bytes(typ, 1 if name == "token_embd.weight" else rows, cols)
    return total


def make_tensor(name, typ, rows, cols, seed):
    """Deterministic content of one tensor: (type, ndarray) — uint8 [nblocks, bb] or float32 [cols]."""
    rng = np.random.default_rng([seed, abs(hash_name(name))])
    if typ == F32:
        return (1.0 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
    if name == "token_embd.weight":
        std = 1.0
    else:
        std = 1.0 / np.sqrt(cols)
    return random_blocks(typ, rows * cols // BLOCK_ELEMS[typ], rng, w_std=std)


def hash_name(name):
    h = 2166136261
    for ch in name.encode():
        h = ((h ^ ch) * 16777619) & 0xFFFFFFFF
    return h


def build_model(shape, mix="q4_k_m", seed=42):
    """(cfg, {name: (type, array, rows, cols)}) fully materialised in host memory."""
    cfg = dict(SHAPES[shape]) if isinstance(shape, str) else dict(shape)
    tensors = {}
    for name, typ, rows, cols in tensor_plan(cfg, mix):
        tensors[name] = (typ, make_tensor(name, typ, rows, cols, seed), rows, cols)
    return cfg, tensors


# ---- GGUF v3 writer ----------------------------------------------------------------------------
def _gs(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _kv_u32(k, v):
    return _gs(k) + struct.pack("<II", 4, v)


def _kv_f32(k, v):
    return _gs(k) + struct.pack("<If", 6, v)


def _kv_str(k, v):
    return _gs(k) + struct.pack("<I", 8) + _gs(v)


def _kv_i32(k, v):
    return _gs(k) + struct.pack("<Ii", 5, v)


def _gb(b):
    return struct.pack("<Q", len(b)) + bytes(b)


def tokenizer_kvs(tokens, model="llama", merges=None, scores=None, token_types=None, bos=None, eos=None, unk=None,
                  pad=None, chat_template=None, vocab_size=None):
    """The tokenizer.* metadata the reference reads (gguf_parser.cpp:240-300, model_config.cpp:199-253). `tokens`,
    `merges`, `chat_template` are bytes (token texts need not be UTF-8)."""
    kvs = [_kv_str("tokenizer.ggml.model", model),
           _gs("tokenizer.ggml.tokens") + struct.pack("<IIQ", 9, 8, len(tokens)) + b"".join(_gb(t) for t in tokens)]
    if merges is not None:
        kvs.append(_gs("tokenizer.ggml.merges") + struct.pack("<IIQ", 9, 8, len(merges)) + b"".join(_gb(m) for m in merges))
    if scores is not None:
        kvs.append(_gs("tokenizer.ggml.scores") + struct.pack("<IIQ", 9, 6, len(scores)) +
                   np.asarray(scores, np.float32).tobytes())
    if token_types is not None:
        kvs.append(_gs("tokenizer.ggml.token_type") + struct.pack("<IIQ", 9, 5, len(token_types)) +
                   np.asarray(token_types, np.int32).tobytes())
    for key, v in (("bos_token_id", bos), ("eos_token_id", eos), ("unk_token_id", unk), ("padding_token_id", pad)):
        if v is not None:
            kvs.append(_kv_i32("tokenizer.ggml." + key, v))
    if chat_template is not None:
        kvs.append(_gs("tokenizer.chat_template") + struct.pack("<I", 8) + _gb(chat_template))
    if vocab_size is not None:
        kvs.append(_kv_u32("tokenizer.ggml.vocab_size", vocab_size))
    return kvs


def write_metadata_gguf(path, kvs, architecture="llama"):
    """A GGUF v3 file with metadata only (no tensors): what the tokenizer tests open."""
    kvs = [_kv_str("general.architecture", architecture)] + list(kvs)
    with open(path, "wb") as f:
        f.write(struct.pack("<IIQQ", 0x46554747, 3, 0, len(kvs)) + b"".join(kvs))
    return path


def write_gguf(path, cfg, tensors, alignment=32, extra_kvs=()):
    """Write `tensors` ({name: (type, array, rows, cols)}) with the metadata keys the reference reads
    (model_config.cpp:149-221). ggml dim order: dims[0] = cols (in_features), dims[1] = rows."""
    kvs = [
        _kv_str("general.architecture", "llama"),
        _kv_str("general.name", "synthetic"),
        _kv_u32("general.alignment", alignment),
        _kv_u32("llama.embedding_length", cfg["hidden"]),
        _kv_u32("llama.feed_forward_length", cfg["inter"]),
        _kv_u32("llama.attention.head_count", cfg["n_heads"]),
        _kv_u32("llama.attention.head_count_kv", cfg["n_kv_heads"]),
        _kv_u32("llama.block_count", cfg["n_layers"]),
        _kv_u32("llama.context_length", cfg["max_pos"]),
        _kv_u32("llama.vocab_size", cfg["vocab"]),
        _kv_f32("llama.attention.layer_norm_rms_epsilon", cfg["eps"]),
        _kv_f32("llama.rope.freq_base", cfg["rope_theta"]),
    ]
    if not extra_kvs:
        kvs += [_kv_u32("tokenizer.ggml.bos_token_id", 1), _kv_u32("tokenizer.ggml.eos_token_id", 2)]
    kvs += list(extra_kvs)
    infos, offset, order = [], 0, []
    for name, (typ, arr, rows, cols) in tensors.items():
        nbytes = arr.nbytes
        dims = [cols] if typ == F32 and rows == 1 else [cols, rows]
        info = _gs(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        info += struct.pack("<IQ", typ, offset)
        infos.append(info)
        order.append((arr, offset))
        offset = (offset + nbytes + alignment - 1) // alignment * alignment
    head = struct.pack("<IIQQ", 0x46554747, 3, len(infos), len(kvs)) + b"".join(kvs) + b"".join(infos)
    pad = (-len(head)) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        start = f.tell()
        for arr, off in order:
            f.seek(start + off)
            f.write(np.ascontiguousarray(arr).tobytes())
        end = start + offset
        f.seek(0, 2)
        if f.tell() < end:
            f.write(b"\0" * (end - f.tell()))
    return path


# ---- layer-list models (tl_model_create_stack): random-init checkpoints in their on-disk form (config.json + safetensors) ----
def to_bf16(a):
    """float32 array -> uint16 array of its bf16 bits (round to nearest even)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def from_bf16(b):
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def stack_layer(heads, kv_heads, dim, vdim, window, v_mix=True, experts=4, top=2, ff=32, shared_ff=64, limit=1.0,
                shared_limit=1.0, scale=None, mlp=True):
    """One entry of config.json's "layers" list. window None: no mask entry (every earlier position is seen)."""
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": float(scale if scale is not None else dim ** -0.5),
             "v_mix": bool(v_mix), "vdim": vdim}
    if window is not None:
        mixer["mask"] = {"size": int(window)}
    ml = None
    if mlp:
        ml = {"kind": "moe", "expert": {"ff": ff, "limit": float(limit)}, "router": {"experts": experts, "top": top},
              "shared": {"ff": shared_ff, "limit": float(shared_limit)} if shared_ff else None}
    return {"type": "attention", "mixer": mixer, "mlp": ml}


def stack_config(width, vocab, layers, eps=1e-5):
    return {"architecture": "Ralasun", "layers": list(layers), "norm": {"eps": float(eps)}, "vocab": int(vocab),
            "width": int(width)}


def build_stack(config, seed=0, gain=1.0):
    """Random tensors {checkpoint name: uint16 bf16 bits}. Projections have std gain / sqrt(fan_in); norm weights are small
    values around zero (the norms apply 1 + w), query/key norm weights around one, router biases of the size of the logits'
    spread, mixing coefficients in (0.2, 0.8)."""
    rng = np.random.default_rng(seed)
    W, V = config["width"], config["vocab"]
    t = {}

    def mat(name, rows, cols, std=None):
        t[name] = to_bf16(rng.standard_normal((rows, cols)).astype(np.float32) * (std or gain / np.sqrt(cols)))

    def vec(name, n, centre, spread):
        t[name] = to_bf16((centre + spread * rng.standard_normal(n)).astype(np.float32))

    mat("embed", V, W, 1.0)
    vec("embed.norm", W, 0.0, 0.1)
    vec("final.norm", W, 0.0, 0.1)
    mat("head", V, W)
    for i, L in enumerate(config["layers"]):
        mx, ml, p = L["mixer"], L.get("mlp"), f"l{i}."
        H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        vec(p + "norm1", W, 0.0, 0.1)
        mat(p + "mix.q", H * d, W)
        mat(p + "mix.k", G * d, W)
        mat(p + "mix.v", G * dv, W)
        mat(p + "mix.o", W, H * dv)
        vec(p + "mix.q.norm", H * d, 1.0, 0.2)
        vec(p + "mix.k.norm", G * d, 1.0, 0.2)
        if mx.get("v_mix"):
            t[p + "mix.vmix"] = to_bf16(np.array(rng.uniform(0.2, 0.8), np.float32))
        if ml is not None:
            vec(p + "norm2", W, 0.0, 0.1)
            E, ff = ml["router"]["experts"], ml["expert"]["ff"]
            mat(p + "mlp.router", E, W)
            vec(p + "mlp.router.b", E, 0.0, 0.5)
            for e in range(E):
                mat(p + f"mlp.e{e}.gate", ff, W, 2.0 / np.sqrt(W))
                mat(p + f"mlp.e{e}.up", ff, W, 2.0 / np.sqrt(W))
                mat(p + f"mlp.e{e}.down", W, ff)
            if ml.get("shared"):
                sff = ml["shared"]["ff"]
                mat(p + "mlp.shared.gate", sff, W, 2.0 / np.sqrt(W))
                mat(p + "mlp.shared.up", sff, W, 2.0 / np.sqrt(W))
                mat(p + "mlp.shared.down", W, sff)
    return t


def madalorn_attention(heads, kv_heads, dim, window=None, keep_first=0, rot_dims=None, base=10000.0, scaling=None, scale=None):
    """The "mixer" entry of a Madalorn attention layer (values are the keys: vdim = dim). scaling: None or a dict
    {factor, original, fast, slow}."""
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": dim,
             "scale": float(scale if scale is not None else dim ** -0.5),
             "rot": {"base": float(base), "dims": int(dim if rot_dims is None else rot_dims)}}
    if scaling:
        mixer["rot"]["scaling"] = {k: (int(v) if k == "original" else float(v)) for k, v in scaling.items()}
    if window is not None:
        mixer["mask"] = {"size": int(window), "keep_first": int(keep_first)}
    return mixer


def madalorn_delta(heads, kv_heads, dim, vdim, conv=4):
    return {"conv": int(conv), "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}


def madalorn_moe(experts, top, ff, shared_ff=0, groups=1, keep=1):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}},
            "shared": {"ff": shared_ff} if shared_ff else None}


def madalorn_layer(kind, mixer, mlp=None, weights_of=None):
    L = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        L["weights_of"] = int(weights_of)
    return L


def madalorn_config(width, vocab, layers, eps=1e-6, softcap=30.0):
    return {"architecture": "Madalorn", "layers": list(layers), "logit_softcap": float(softcap), "norm": {"eps": float(eps)},
            "vocab": int(vocab), "width": int(width)}


def build_madalorn(config, seed=0, gain=1.0, ranks=(8, 8)):
    """Random tensors {checkpoint name: uint16 bf16 bits} of a Madalorn configuration. Layers with weights_of get none.
    ranks: inner sizes of the decay and output-gate projections of delta layers."""
    rng = np.random.default_rng(seed)
    W, V = config["width"], config["vocab"]
    t = {}

    def mat(name, rows, cols, std=None):
        t[name] = to_bf16(rng.standard_normal((rows, cols)).astype(np.float32) * (std or gain / np.sqrt(cols)))

    def vec(name, n, centre, spread, shape=None):
        a = to_bf16((centre + spread * rng.standard_normal(n)).astype(np.float32))
        t[name] = a.reshape(shape) if shape is not None else a

    def norm(name):
        vec(name, W, 1.0, 0.1)
        vec(name + ".b", W, 0.0, 0.05)
        t[name + ".alpha"] = to_bf16(np.array(rng.uniform(0.4, 0.9), np.float32)).reshape(())  # a scalar tensor: shape []

    def glu(p, ff):
        mat(p + "gate", ff, W, 2.0 / np.sqrt(W))
        mat(p + "up", ff, W, 2.0 / np.sqrt(W))
        mat(p + "down", W, ff)

    mat("embed", V, W, 1.0)
    norm("final.norm")
    mat("head", V, W, 4.0 / np.sqrt(W))
    for i, L in enumerate(config["layers"]):
        if "weights_of" in L:
            continue
        mx, ml, p = L["mixer"], L.get("mlp"), f"l{i}."
        H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        norm(p + "norm1")
        if L["type"] == "attention":
            mat(p + "mix.q", H * d, W)
            mat(p + "mix.k", G * d, W)
            vec(p + "mix.pb", H, -1.0, 0.5)
            mat(p + "mix.o", W, H * dv)
        else:
            ra, rg = ranks
            mat(p + "mix.q", G * d, W)
            mat(p + "mix.k", G * d, W)
            mat(p + "mix.v", H * dv, W)
            for n, c in (("q", G * d), ("k", G * d), ("v", H * dv)):
                mat(p + f"mix.{n}.conv", c, mx["conv"], 0.5)
            mat(p + "mix.b", H, W)
            vec(p + "mix.A_log", H, -0.5, 0.5)
            vec(p + "mix.norm", dv, 1.0, 0.1)
            mat(p + "mix.a1", ra, W)
            mat(p + "mix.a2", H * d, ra)
            vec(p + "mix.dt_bias", H * d, -1.0, 0.5)
            mat(p + "mix.g1", rg, W)
            mat(p + "mix.g2", H * dv, rg)
            mat(p + "mix.o", W, H * dv)
        if ml is None:
            continue
        if ml["kind"] == "dense":
            glu(p + "mlp.", ml["ff"])
        else:
            E = ml["router"]["experts"]
            for e in range(E):
                glu(p + f"mlp.e{e}.", ml["expert"]["ff"])
            mat(p + "mlp.router", E, W, 2.0 / np.sqrt(W))
            if ml.get("shared"):
                glu(p + "mlp.shared.", ml["shared"]["ff"])
                mat(p + "mlp.shared.sg", 1, W)
    return t


def sogalix_attention(heads, kv_heads, dim, vdim, q_temp=None, scale=None):
    """The "mixer" entry of a Sogalix attention layer; q_temp: None or (coef, every)."""
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "scale": float(scale if scale is not None else dim ** -0.5)}
    if q_temp is not None:
        mixer["q_temp"] = {"coef": float(q_temp[0]), "every": int(q_temp[1])}
    return mixer


def sogalix_latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=10000.0, kv_from=None, scale=None):
    mixer = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot": {"base": float(base), "dims": rot_dim},
             "rot_dim": rot_dim, "scale": float(scale if scale is not None else (dim + rot_dim) ** -0.5), "vdim": vdim}
    if kv_from is not None:
        mixer["kv_from"] = int(kv_from)
    return mixer


def sogalix_delta(heads, dim):
    return {"dim": dim, "heads": heads}


def sogalix_layer(kind, mixer, ff=None):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": int(ff)} if ff else None}


def sogalix_config(width, vocab, layers, eps=1e-6):
    return {"architecture": "Sogalix", "layers": list(layers), "norm": {"eps": float(eps)}, "vocab": int(vocab), "width": int(width)}


def build_sogalix(config, seed=0, gain=1.0, decay_rank=8):
    """Random tensors {checkpoint name: uint16 bf16 bits} of a Sogalix configuration. decay_rank: inner size of the
    generalized delta rule's two-step decay projection (the configuration does not name it; the tensors' shapes do)."""
    rng = np.random.default_rng(seed)
    W, V = config["width"], config["vocab"]
    t = {}

    def mat(name, rows, cols, std=None):
        t[name] = to_bf16(rng.standard_normal((rows, cols)).astype(np.float32) * (std or gain / np.sqrt(cols)))

    def vec(name, n, centre, spread):
        t[name] = to_bf16((centre + spread * rng.standard_normal(n)).astype(np.float32))

    def norm(name):
        vec(name, W, 1.0, 0.1)
        vec(name + ".b", W, 0.0, 0.05)

    mat("embed", V, W, 1.0)
    norm("embed.norm")
    norm("final.norm")
    mat("head", V, W, 4.0 / np.sqrt(W))
    for i, L in enumerate(config["layers"]):
        mx, ml, p = L["mixer"], L.get("mlp"), f"l{i}."
        H, d = mx["heads"], mx["dim"]
        norm(p + "norm1")
        if L["type"] == "attention":
            G, dv = mx["kv_heads"], mx["vdim"]
            mat(p + "mix.q", H * d, W, 2.0 / np.sqrt(W))
            mat(p + "mix.k", G * d, W, 2.0 / np.sqrt(W))
            mat(p + "mix.v", G * dv, W)
            mat(p + "mix.o", W, H * dv)
        elif L["type"] == "latent_attention":
            rd, dv, rq, rk = mx["rot_dim"], mx["vdim"], mx["q_rank"], mx["kv_rank"]
            mat(p + "mix.dq", rq, W)
            vec(p + "mix.dq.norm", rq, 1.0, 0.1)
            mat(p + "mix.uq", H * (d + rd), rq, 2.0 / np.sqrt(rq))
            if mx.get("kv_from") is None:
                mat(p + "mix.dkv", rk + rd, W)
                vec(p + "mix.dkv.norm", rk, 1.0, 0.1)
            mat(p + "mix.uk", H * d, rk, 2.0 / np.sqrt(rk))
            mat(p + "mix.uv", H * dv, rk)
            mat(p + "mix.g", H, W, 2.0 / np.sqrt(W))
            mat(p + "mix.o", W, H * dv)
        else:
            for n in "rkvga":
                mat(p + "mix." + n, H * d, W)
            vec(p + "mix.a.b", H * d, 0.0, 0.5)
            mat(p + "mix.w1", decay_rank, W, 2.0 / np.sqrt(W))
            mat(p + "mix.w2", H * d, decay_rank, 1.0)
            vec(p + "mix.w0", H * d, -1.0, 1.0)
            vec(p + "mix.norm", H * d, 1.0, 0.1)
            mat(p + "mix.o", W, H * d)
        if ml is not None:
            norm(p + "norm2")
            mat(p + "mlp.up", ml["ff"], W, 2.0 / np.sqrt(W))
            mat(p + "mlp.down", W, ml["ff"])
            t[p + "mlp.act"] = to_bf16(np.array([rng.uniform(-1.0, 1.0), rng.uniform(-1.0, 1.0)], np.float32))
    return t


def potipel_attention(heads, kv_heads, dim, vdim, diff=0.5, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": float(diff),
            "scale": float(scale if scale is not None else dim ** -0.5)}


def potipel_hgrn2(heads, dim, vdim):
    return {"heads": heads, "dim": dim, "vdim": vdim}


def potipel_pair(left_heads, left_kv_heads, left_dim, left_vdim, window, heads, kv_heads, dim, vdim, conv=4, right_conv=None,
                 softcap=20.0, left_scale=1.0, right_scale=1.0, scale=None):
    left = {"heads": left_heads, "kv_heads": left_kv_heads, "dim": left_dim, "vdim": left_vdim, "conv": conv,
            "softcap": float(softcap), "scale": float(scale if scale is not None else left_dim ** -0.5)}
    if window:
        left["mask"] = {"size": int(window)}
    right = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": right_conv or conv}
    return {"left": left, "right": right, "left_scale": float(left_scale), "right_scale": float(right_scale)}


def potipel_moe(experts, top, ff, groups=1, keep=1, limit=1.5):
    return {"kind": "moe", "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}},
            "expert": {"ff": ff, "limit": float(limit)}}


def potipel_layer(kind, mixer, mlp=None, weights_of=None):
    """kind: "attention" | "hgrn2" | "parallel"; mlp: None, an int (the relu-gated unit's size) or potipel_moe(...)."""
    L = {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": mlp} if isinstance(mlp, int) else mlp}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def potipel_config(width, vocab, layers, eps=1e-6, embed_scale=4.0, taps=3):
    return {"architecture": "Potipel", "canon": {"taps": int(taps)}, "embedding": {"scale": float(embed_scale)},
            "layers": list(layers), "norm": {"eps": float(eps)}, "vocab": int(vocab), "width": int(width)}


def build_potipel(config, seed=0, gain=1.0):
    """Random tensors {checkpoint name: uint16 bf16 bits} of a Potipel configuration (a layer with weights_of has none)."""
    rng = np.random.default_rng(seed)
    W, V, taps = config["width"], config["vocab"], config["canon"]["taps"]
    t = {}

    def mat(name, rows, cols, std=None):
        t[name] = to_bf16(rng.standard_normal((rows, cols)).astype(np.float32) * (std or gain / np.sqrt(cols)))

    def vec(name, n, centre, spread):
        t[name] = to_bf16((centre + spread * rng.standard_normal(n)).astype(np.float32))

    mat("embed", V, W, 1.0 / config["embedding"]["scale"])
    vec("final.norm", W, 1.0, 0.1)
    mat("head", V, W, 4.0 / np.sqrt(W))
    for i, L in enumerate(config["layers"]):
        if "weights_of" in L:
            continue
        mx, ml, p = L["mixer"], L.get("mlp"), f"l{i}."
        vec(p + "norm1", W, 1.0, 0.1)
        mat(p + "canon1", W, taps, 0.3)
        if L["type"] == "attention":
            H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            mat(p + "mix.q", H * 2 * d, W, 2.0 / np.sqrt(W))
            mat(p + "mix.k", G * 2 * d, W, 2.0 / np.sqrt(W))
            mat(p + "mix.v", G * dv, W)
            vec(p + "mix.q.norm", d, 1.5, 0.3)
            vec(p + "mix.k.norm", d, 1.5, 0.3)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                vec(p + "mix." + n, d, 0.0, 0.3)
            mat(p + "mix.g", H * dv, W, 2.0 / np.sqrt(W))
            mat(p + "mix.o", W, H * dv)
        elif L["type"] == "hgrn2":
            H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
            mat(p + "mix.q", H * d, W, 2.0 / np.sqrt(W))
            mat(p + "mix.f", H * d, W, 2.0 / np.sqrt(W))
            vec(p + "mix.f.b", H * d, 1.0, 1.0)
            t[p + "mix.lower"] = to_bf16(rng.uniform(0.0, 0.9, H * d).astype(np.float32))
            mat(p + "mix.v", H * dv, W)
            vec(p + "mix.norm", dv, 1.0, 0.1)
            mat(p + "mix.o", W, H * dv)
        else:
            lt, rt, q = mx["left"], mx["right"], p + "mix.left."
            H, G, d, dv = lt["heads"], lt["kv_heads"], lt["dim"], lt["vdim"]
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
                mat(q + n, rows, W, 2.0 / np.sqrt(W))
                vec(q + n + ".b", rows, 0.0, 0.2)
                mat(q + n + ".conv", rows, lt["conv"], 0.5)
            t[q + "r1"] = to_bf16(rng.uniform(0.2, 1.5, H).astype(np.float32))
            t[q + "r2"] = to_bf16(rng.uniform(0.05, 1.0, H).astype(np.float32))
            vec(q + "sink", H, 0.0, 1.0)
            mat(q + "o", W, H * dv)
            q = p + "mix.right."
            H, G, d, dv = rt["heads"], rt["kv_heads"], rt["dim"], rt["vdim"]
            for n, rows in (("q", G * d), ("k", G * d), ("v", H * dv)):
                mat(q + n, rows, W, 2.0 / np.sqrt(W))
                mat(q + n + ".conv", rows, rt["conv"], 0.5)
            mat(q + "b", H, W, 2.0 / np.sqrt(W))
            mat(q + "a", H, W, 2.0 / np.sqrt(W))
            vec(q + "A_log", H, -1.0, 1.0)
            vec(q + "dt_bias", H, 0.0, 1.0)
            vec(q + "norm", dv, 1.0, 0.1)
            mat(q + "g", H * dv, W, 2.0 / np.sqrt(W))
            mat(q + "o", W, H * dv)
        if ml is not None:
            vec(p + "norm2", W, 1.0, 0.1)
            mat(p + "canon2", W, taps, 0.3)
            if ml["kind"] == "dense":
                mat(p + "mlp.gate", ml["ff"], W, 2.0 / np.sqrt(W))
                mat(p + "mlp.up", ml["ff"], W, 2.0 / np.sqrt(W))
                mat(p + "mlp.down", W, ml["ff"])
            else:
                E, ff = ml["router"]["experts"], ml["expert"]["ff"]
                mat(p + "mlp.router", E, W, 3.0 / np.sqrt(W))
                vec(p + "mlp.correction", E, 0.0, 0.3)
                for e in range(E):
                    mat(f"{p}mlp.e{e}.gate", ff, W, 2.0 / np.sqrt(W))
                    mat(f"{p}mlp.e{e}.up", ff, W, 2.0 / np.sqrt(W))
                    mat(f"{p}mlp.e{e}.down", W, ff)
    return t


def write_stack_dir(path, config, tensors):
    """config.json + model.safetensors (8-byte little-endian header length, JSON header, data) under `path`."""
    import json
    import os
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f, indent=1)
    header, off, blobs = {}, 0, []
    for name, a in tensors.items():
        shape = list(np.shape(a))  # (a scalar tensor keeps its empty shape)
        a = np.ascontiguousarray(a)
        dt = {np.dtype(np.uint16): "BF16", np.dtype(np.float32): "F32", np.dtype(np.int32): "I32"}[a.dtype]
        b = a.tobytes()
        header[name] = {"dtype": dt, "shape": shape, "data_offsets": [off, off + len(b)]}
        off += len(b)
        blobs.append(b)
    h = json.dumps(header, separators=(",", ":")).encode()
    h += b" " * (-len(h) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)
