"""Tensor lists of the five benchmark configurations (names and shapes only, no data).

The shapes follow the models the reference trains:
  * FLUX.1-dev: hidden 3072, 24 heads, 19 double-stream and 38 single-stream blocks, mlp_ratio 4
    (src/models/flux_model_complete.rs:424-441; Attention :244-245, FeedForward :266-267,
    single-stream linear1/linear2 :844-846, embedders :516-547, final layer :579).
  * SDXL UNet: block_out_channels [320, 640, 1280], 2 layers per block, transformer depth
    [1, 2, 10], cross-attention width 2048 (src/models/sdxl_unet_complete.rs:53-96).
  * LoRA adapters: A = [rank, in], B = [out, rank] (src/networks/lora.rs:83,93).
`scale` divides every channel width so the tests can run the same tensor structure at a size a CPU
finishes in seconds.
"""
import random

BLOCK = 2048


def numel(shape):
    n = 1
    for d in shape:
        n *= int(d)
    return n


def total_params(tensors):
    return sum(numel(s) for _, s in tensors)


def total_blocks(tensors):
    return sum((numel(s) + BLOCK - 1) // BLOCK for _, s in tensors)


def c1_flat():
    """Config 1: one flat fp32 tensor of 2**20 elements."""
    return [("flat", (1 << 20,))]


def c2_sdxl_lora(rank=16, pairs=700, seed=0xE21D + 2, scale=1):
    """Config 2: ~700 LoRA pairs with in/out drawn from the SDXL UNet's linear widths."""
    widths = [320, 640, 1280, 2048, 2560, 5120]
    rng = random.Random(seed)
    out = []
    for i in range(pairs):
        fin = max(rng.choice(widths) // scale, 1)
        fout = max(rng.choice(widths) // scale, 1)
        out.append(("lora.%d.down" % i, (rank, fin)))
        out.append(("lora.%d.up" % i, (fout, rank)))
    return out


def _flux_linears(hidden, mlp):
    """(name, in, out) of every linear inside the DiT blocks."""
    lin = []
    for b in range(19):
        for stream in ("img", "txt"):
            pre = "double_blocks.%d.%s" % (b, stream)
            lin += [(pre + "_mod.lin", hidden, 6 * hidden), (pre + "_attn.qkv", hidden, 3 * hidden),
                    (pre + "_attn.proj", hidden, hidden), (pre + "_mlp.0", hidden, mlp),
                    (pre + "_mlp.2", mlp, hidden)]
    for b in range(38):
        pre = "single_blocks.%d" % b
        lin += [(pre + ".modulation.lin", hidden, 3 * hidden),
                (pre + ".linear1", hidden, 3 * hidden + mlp), (pre + ".linear2", hidden + mlp, hidden)]
    return lin


def c3_flux_lora(rank=32, scale=1):
    """Config 3: rank-32 LoRA on every linear of the 19 + 38 DiT blocks (608 tensors)."""
    hidden, mlp = 3072 // scale, 12288 // scale
    out = []
    for name, fin, fout in _flux_linears(hidden, mlp):
        out.append((name + ".lora_A", (rank, fin)))
        out.append((name + ".lora_B", (fout, rank)))
    return out


def c5_flux_full(scale=1):
    """Config 5: every weight, bias and QK-norm scale of a FLUX-12B-shaped model (780 tensors)."""
    hidden, mlp = 3072 // scale, 12288 // scale
    head = max(128 // scale, 1)
    out = []

    def linear(name, fin, fout):
        out.append((name + ".weight", (fout, fin)))
        out.append((name + ".bias", (fout,)))

    linear("img_in", 64, hidden)
    linear("txt_in", max(4096 // scale, 1), hidden)
    for emb, fin in (("time_in", 256), ("vector_in", 768), ("guidance_in", 256)):
        linear(emb + ".in_layer", fin, hidden)
        linear(emb + ".out_layer", hidden, hidden)
    for name, fin, fout in _flux_linears(hidden, mlp):
        linear(name, fin, fout)
        if name.endswith("_attn.qkv"):
            base = name[:-len(".qkv")]
            out.append((base + ".norm.query_norm.scale", (head,)))
            out.append((base + ".norm.key_norm.scale", (head,)))
        if name.endswith(".linear2"):
            base = name[:-len(".linear2")]
            out.append((base + ".norm.query_norm.scale", (head,)))
            out.append((base + ".norm.key_norm.scale", (head,)))
    linear("final_layer.adaLN_modulation.1", hidden, 2 * hidden)
    linear("final_layer.linear", hidden, 64)
    return out


def c4_sdxl_full(scale=1):
    """Config 4: an SDXL-UNet-shaped full parameter set (~1,700 tensors, ~2.6 B parameters)."""
    ch = [320 // scale, 640 // scale, 1280 // scale]
    temb = 1280 // scale
    ctx = 2048 // scale
    depth = [1, 2, 10]
    out = []

    def conv(name, cin, cout, k=3):
        out.append((name + ".weight", (cout, cin, k, k)))
        out.append((name + ".bias", (cout,)))

    def linear(name, fin, fout, bias=True):
        out.append((name + ".weight", (fout, fin)))
        if bias:
            out.append((name + ".bias", (fout,)))

    def norm(name, c):
        out.append((name + ".weight", (c,)))
        out.append((name + ".bias", (c,)))

    def resnet(name, cin, cout):
        norm(name + ".norm1", cin)
        conv(name + ".conv1", cin, cout)
        linear(name + ".time_emb_proj", temb, cout)
        norm(name + ".norm2", cout)
        conv(name + ".conv2", cout, cout)
        if cin != cout:
            conv(name + ".conv_shortcut", cin, cout, 1)

    def transformer(name, c, layers):
        norm(name + ".norm", c)
        linear(name + ".proj_in", c, c)
        for i in range(layers):
            pre = "%s.transformer_blocks.%d" % (name, i)
            norm(pre + ".norm1", c)
            for w in ("to_q", "to_k", "to_v"):
                linear(pre + ".attn1." + w, c, c, bias=False)
            linear(pre + ".attn1.to_out.0", c, c)
            norm(pre + ".norm2", c)
            linear(pre + ".attn2.to_q", c, c, bias=False)
            linear(pre + ".attn2.to_k", ctx, c, bias=False)
            linear(pre + ".attn2.to_v", ctx, c, bias=False)
            linear(pre + ".attn2.to_out.0", c, c)
            norm(pre + ".norm3", c)
            linear(pre + ".ff.net.0.proj", c, 8 * c)
            linear(pre + ".ff.net.2", 4 * c, c)
        linear(name + ".proj_out", c, c)

    conv("conv_in", 4, ch[0])
    linear("time_embedding.linear_1", ch[0], temb)
    linear("time_embedding.linear_2", temb, temb)
    linear("add_embedding.linear_1", max(2816 // scale, 1), temb)
    linear("add_embedding.linear_2", temb, temb)
    prev = ch[0]
    for b, c in enumerate(ch):
        for j in range(2):
            resnet("down_blocks.%d.resnets.%d" % (b, j), prev if j == 0 else c, c)
            if b > 0:
                transformer("down_blocks.%d.attentions.%d" % (b, j), c, depth[b])
        prev = c
        if b < 2:
            conv("down_blocks.%d.downsamplers.0.conv" % b, c, c)
    resnet("mid_block.resnets.0", ch[2], ch[2])
    transformer("mid_block.attentions.0", ch[2], depth[2])
    resnet("mid_block.resnets.1", ch[2], ch[2])
    skip = [ch[0], ch[0], ch[0], ch[0], ch[1], ch[1], ch[1], ch[2], ch[2]]  # down-path outputs
    prev = ch[2]
    for b, c in enumerate(reversed(ch)):
        lvl = 2 - b
        for j in range(3):
            cin = prev + skip.pop()
            resnet("up_blocks.%d.resnets.%d" % (b, j), cin, c)
            prev = c
            if lvl > 0:
                transformer("up_blocks.%d.attentions.%d" % (b, j), c, depth[lvl])
        if b < 2:
            conv("up_blocks.%d.upsamplers.0.conv" % b, c, c)
    norm("conv_norm_out", ch[0])
    conv("conv_out", ch[0], 4)
    return out


def init_std(config, name, shape):
    """(standard deviation of the parameters, of the gradients) the benchmark configuration names for a tensor.
    LoRA sets: A ~ N(0, 1/in), B zero-initialised then perturbed ~ N(0, 1e-4), gradients ~ N(0, 1e-4); the flat
    tensor and the full fine-tune sets: parameters ~ N(0, 0.02), gradients ~ N(0, 1e-3)."""
    if config in ("c2_sdxl_lora_r16", "c3_flux_lora_r32"):
        is_a = name.endswith(".down") or name.endswith(".lora_A")
        return (float(shape[1]) ** -0.5 if is_a else 1e-4), 1e-4
    return 0.02, 1e-3


CONFIGS = {
    "c1_flat_fp32": (c1_flat, "f32"),
    "c2_sdxl_lora_r16": (c2_sdxl_lora, "bf16"),
    "c3_flux_lora_r32": (c3_flux_lora, "bf16"),
    "c4_sdxl_unet_full": (c4_sdxl_full, "bf16"),
    "c5_flux12b_full": (c5_flux_full, "bf16"),
}
