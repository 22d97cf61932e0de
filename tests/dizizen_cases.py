"""Small Dizizen configurations for the tests: sizes, constants and orders of layers that differ in every way the design allows."""


def dense(ff=48, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts=6, identity=0, top=2, groups=None, ff=16, shared=None):
    router = {"experts": experts, "top": top}
    if identity:
        router["identity"] = identity
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def layer(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.25, rot=(8, 10000.0), kv_from=None, mlp="dense"):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"dims": rot[0], "base": rot[1]}}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": dense() if mlp == "dense" else mlp}


def model(layers, width=64, vocab=97, eps=1e-5, mult=0.5, embedding_scale=8.0):
    return {"architecture": "Dizizen", "embedding": {"scale": embedding_scale}, "layers": layers, "norm": {"eps": eps}, "residual_mult": mult,
            "vocab": vocab, "width": width}


CASES = {
    # every kind of feed-forward and none; a layer that borrows keys and values two layers back and one right behind its source; grouped
    # heads; rotation of a part of a head; groups of experts with and without experts that hand their input on; a shared expert
    "mixed": model([
        layer(),
        layer(heads=2, kv_heads=2, dim=24, vdim=16, scale=0.2, rot=(24, 100.0), mlp=moe(experts=6, identity=2, top=3, groups=(4, 2), ff=16, shared=24)),
        layer(kv_from=0, mlp=None),
        layer(heads=2, kv_heads=2, dim=24, vdim=16, scale=0.2, rot=(24, 100.0), kv_from=1, mlp=moe(experts=5, top=1, ff=24)),
        layer(heads=2, kv_heads=1, dim=16, vdim=32, scale=0.3, rot=(4, 500.0), mlp=dense(ff=40, limit=0.4)),
    ]),
    # sizes that are no multiples of anything a kernel would like; one key/value head; a single group; as many picked as there are experts
    # in the kept groups; only the shared expert has more units than the routed ones; a multiplier of 1
    "odd": model([
        layer(heads=5, kv_heads=1, dim=20, vdim=12, scale=0.3, rot=(6, 777.0), mlp=moe(experts=3, identity=1, top=2, groups=(2, 1), ff=10, shared=50)),
        layer(heads=3, kv_heads=3, dim=10, vdim=36, scale=0.35, rot=(10, 50.0), mlp=dense(ff=90, limit=3.0)),
        layer(heads=6, kv_heads=3, dim=10, vdim=36, scale=0.2, rot=(10, 50.0), kv_from=1, mlp=moe(experts=7, top=3, ff=12)),
        layer(heads=5, kv_heads=1, dim=20, vdim=12, scale=0.3, rot=(6, 777.0), kv_from=0, mlp=None),
    ], width=100, vocab=77, eps=1e-6, mult=1.0, embedding_scale=10.0),
    # heads of powers of two (the split-key kernel decodes them and the streaming kernel takes their prompts), four query heads to a
    # key/value head, as many query as key/value heads, values wider and narrower than keys, no rotation of queries and keys at all
    "wide": model([
        layer(heads=4, kv_heads=1, dim=32, vdim=64, scale=0.18, rot=(16, 10000.0), mlp=dense(ff=96, limit=1.0)),
        layer(heads=2, kv_heads=2, dim=64, vdim=32, scale=0.125, rot=(0, 500.0), mlp=moe(experts=8, identity=4, top=4, groups=(3, 2), ff=32)),
        layer(heads=4, kv_heads=1, dim=32, vdim=64, scale=0.18, rot=(16, 10000.0), kv_from=0, mlp=moe(experts=4, top=2, groups=(2, 2), ff=32, shared=32)),
        layer(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.2, rot=(32, 500.0), mlp=None),
    ], width=96, vocab=130, mult=0.3, embedding_scale=9.8),
    # heads of 80 to 192 (pages of 96, 128 and 192 elements a head: other attention kernels than heads of 64 take)
    "large": model([
        layer(heads=4, kv_heads=2, dim=80, vdim=96, scale=80 ** -0.5, rot=(40, 20000.0), mlp=dense(ff=200, limit=2.0)),
        layer(heads=2, kv_heads=1, dim=128, vdim=192, scale=128 ** -0.5, rot=(128, 300.0), mlp=moe(experts=4, identity=2, top=2, groups=(3, 2), ff=64, shared=64)),
        layer(heads=2, kv_heads=1, dim=128, vdim=192, scale=0.1, rot=(128, 300.0), kv_from=1, mlp=None),
    ], width=160, vocab=211, mult=0.7, embedding_scale=12.6),
}
