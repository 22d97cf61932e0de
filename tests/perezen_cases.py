"""Small Perezen configurations for the tests: sizes, constants and orders of layers that differ in every way the design allows."""


def mlp(ff):
    return None if ff is None else {"kind": "dense", "ff": ff}


def mlstm_layer(heads=2, dim=16, vdim=24, cap=8.0, ff=None):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim}
    if cap is not None:
        mixer["gate_cap"] = cap
    return {"type": "mlstm", "mixer": mixer, "mlp": mlp(ff)}


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.25, diff=0.4, chunk=40, rot=(8, 10000.0), kv_from=None, ff=48):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if chunk is not None:
        mixer["mask"] = {"size": chunk}
    if rot is not None:
        mixer["rot"] = {"dims": rot[0], "base": rot[1]}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": mlp(ff)}


def model(layers, width=64, vocab=97, eps=1e-5, logit_scale=1.0, max_positions=320):
    return {"architecture": "Perezen", "layers": layers, "logit_scale": logit_scale, "max_positions": max_positions, "norm": {"eps": eps},
            "vocab": vocab, "width": width}


CASES = {
    # both kinds of layer, with and without a feed-forward; a layer that borrows keys and values and looks through other chunks at them;
    # grouped heads; chunks shorter and longer than a page and none; rotation of a part of a map, of all of it and none
    "mixed": model([
        attention_layer(),
        mlstm_layer(),
        attention_layer(chunk=100, rot=(8, 10000.0), kv_from=0, diff=0.7, ff=None),
        attention_layer(heads=2, kv_heads=2, dim=24, vdim=16, chunk=None, rot=(24, 100.0), scale=0.2, diff=0.1),
        mlstm_layer(heads=3, dim=8, vdim=8, cap=None, ff=48),
        attention_layer(heads=2, kv_heads=1, dim=16, vdim=32, chunk=70, rot=None, diff=0.25, ff=None),
        attention_layer(heads=2, kv_heads=1, dim=16, vdim=32, chunk=None, rot=None, kv_from=5, diff=0.5),
    ], logit_scale=1.7),
    # sizes that are no multiples of anything a kernel would like; a matrix memory first; one key/value head; chunks of five
    "odd": model([
        mlstm_layer(heads=5, dim=20, vdim=12, cap=3.0, ff=90),
        attention_layer(heads=5, kv_heads=1, dim=20, vdim=12, scale=0.3, diff=0.6, chunk=5, rot=(6, 777.0), ff=90),
        attention_layer(heads=3, kv_heads=3, dim=10, vdim=36, scale=0.35, diff=0.3, chunk=33, rot=(10, 50.0), ff=None),
        attention_layer(heads=6, kv_heads=3, dim=10, vdim=36, scale=0.2, diff=0.45, chunk=64, rot=(10, 50.0), kv_from=2),
    ], width=100, vocab=77, eps=1e-6, logit_scale=0.5, max_positions=300),
    # heads of powers of two (the split-key kernel decodes them and the streaming kernel takes their prompts), a chunk of exactly one page
    # and one of two, four query heads to a key/value head, as many query as key/value heads
    "wide": model([
        attention_layer(heads=4, kv_heads=1, dim=32, vdim=64, scale=0.18, diff=0.5, chunk=64, rot=(16, 10000.0), ff=96),
        mlstm_layer(heads=2, dim=64, vdim=64, cap=12.0),
        attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.2, diff=0.35, chunk=128, rot=(32, 500.0)),
        attention_layer(heads=4, kv_heads=1, dim=32, vdim=64, scale=0.18, diff=0.2, chunk=96, rot=(16, 10000.0), kv_from=0, ff=None),
    ], width=96, vocab=130, logit_scale=2.0, max_positions=400),
    # heads of 80 to 192 (pages of 96, 128 and 192 elements a head: other attention kernels than heads of 64 take), a matrix memory of 96 x 128
    "large": model([
        attention_layer(heads=4, kv_heads=2, dim=80, vdim=96, scale=80 ** -0.5, diff=0.5, chunk=100, rot=(40, 20000.0)),
        mlstm_layer(heads=2, dim=96, vdim=128, cap=10.0),
        attention_layer(heads=2, kv_heads=1, dim=128, vdim=192, scale=128 ** -0.5, diff=0.3, chunk=150, rot=(128, 300.0), ff=None),
        attention_layer(heads=2, kv_heads=1, dim=64, vdim=128, scale=0.125, diff=0.6, chunk=None, rot=(32, 5000.0), ff=200),
    ], width=160, vocab=211, max_positions=300),
}
