"""Small driver for rocprofv3 runs: launches each hot kernel of configuration 2
(and 4) a few times, plus a plain device copy of known size that calibrates the
FETCH_SIZE / WRITE_SIZE counters.

    rocprofv3 --kernel-trace --stats -d OUT -o kt --output-format csv -- python3 profile_kernels.py
    rocprofv3 --pmc FETCH_SIZE -d OUT -o fetch --output-format csv -- python3 profile_kernels.py
    rocprofv3 --pmc WRITE_SIZE -d OUT -o write --output-format csv -- python3 profile_kernels.py

With the argument ``around-attention`` it launches instead the kernels either side of the ring
step: the attention core at head size 128 (32 heads, 4096 x 4096 tokens) and the qkv / output
projections with the head split fused in (8 x 4096 tokens, 512 channels, 8 heads). With
``swin-block`` it runs forward + backward of one Swin block on a 256 x 256 token tile (dim 128,
4 heads, 8 x 8 windows, shift 4, bf16 autocast; the neighbours' roll slabs are random stand-ins made once).
With ``sharded-layernorm`` it runs forward + backward of the channel-sharded LayerNorm on one shard's
rows, bf16, at configuration 4's local width and at a row count that fills the chip (2 ** 18 rows of
256 channels), then at 2 ** 20 rows of 64 channels and, for the kernels that walk a row, of 132.
With ``attention-fp32`` it runs the attention core forward + backward on fp32 inputs (8 heads,
4096 x 4096 tokens) at head sizes 64, 128 and 32.
"""

from __future__ import annotations

import sys

import torch


def main(reps: int = 3) -> None:
    from jigsaw_amd import attention as ja
    from jigsaw_amd import conv as jc
    from jigsaw_amd.halo import HaloGeometry, halo_assemble, halo_fold, halo_fold_border_, halo_pack

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    batch, ch, tile = 8, 64, 1024
    geom = HaloGeometry((tile, tile), (1, 1), (1, 1))
    lead = (batch, ch)
    x = torch.randn(*lead, tile, tile, device=dev, generator=g).bfloat16()
    w = ((torch.rand(ch, ch, 3, 3, device=dev, generator=g) * 2 - 1) / 24).bfloat16()
    b = ((torch.rand(ch, device=dev, generator=g) * 2 - 1) / 24).bfloat16()
    gout = torch.randn(*lead, tile, tile, device=dev, generator=g).bfloat16()
    sf = {o: torch.randn(*lead, *geom.strip_extent(o, "assemble"), device=dev, generator=g).bfloat16() for o in geom.offsets()}
    sb = {o: torch.randn(*lead, *geom.strip_extent(o, "fold"), device=dev, generator=g).bfloat16() for o in geom.offsets()}
    x_aug = halo_assemble(x, sf, geom)
    gx_aug = jc.conv_nd_input(x_aug.shape, w, gout)
    gx = torch.empty_like(x)
    copy_dst = torch.empty_like(x)  # calibration copy: reads and writes x.numel() * 2 bytes
    q = (torch.randn(1, 8, 4096, 64, device=dev, generator=g) / 8).bfloat16()
    k = torch.randn(1, 8, 4096, 64, device=dev, generator=g).bfloat16()
    v = torch.randn(1, 8, 4096, 64, device=dev, generator=g).bfloat16()
    acc = torch.zeros(1, 8, 4096, 64, device=dev)
    lse = torch.full((1, 8, 4096), float("-inf"), device=dev)
    out, l = ja.core_forward(q, k, v, 0.125)
    for _ in range(reps):
        copy_dst.copy_(x)
        # the step as the benchmark runs it (fused backward)
        halo_pack(x, geom, from_padded=False)
        halo_assemble(x, sf, geom, out=x_aug)
        jc.conv_nd(x_aug, w, b)
        gx_f, _send = jc.conv_nd_input_fold(geom, w, gout)
        jc.conv_nd_weight(x_aug, w.shape, gout, with_bias_grad=True)
        halo_fold_border_(gx_f, sb, geom)
        # the separate steps the fused ones replace
        jc.conv_nd_input(x_aug.shape, w, gout)
        jc.sum_grad_bias(gout, 2)
        halo_fold(gx_aug, sb, geom, out=gx)
        ja.core_forward(q, k, v, 0.125, out_acc=acc, lse_acc=lse, want_out=False)
        ja.core_backward(gout[0, :8, :, :64].reshape(1, 8, 1024 * 1, 64).expand(1, 8, 1024, 64).repeat(1, 1, 4, 1), q, k, v, out, l, 0.125)
    torch.cuda.synchronize()
    print("profile_kernels: done", file=sys.stderr)


def around_attention(reps: int = 3) -> None:
    from jigsaw_amd import attention as ja
    from jigsaw_amd import projection as jp

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(1)
    h, n, d = 32, 4096, 128
    q = (torch.randn(1, h, n, d, device=dev, generator=g) / d**0.5).bfloat16()
    k = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    v = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    dout = torch.randn(1, h, n, d, device=dev, generator=g).bfloat16()
    out, lse = ja.core_forward(q, k, v, d**-0.5)
    bsz, c, heads = 8, 512, 8
    x = torch.randn(bsz, n, c, device=dev, generator=g).bfloat16().requires_grad_()
    w = (torch.randn(3 * c, c, device=dev, generator=g) / c**0.5).bfloat16().requires_grad_()
    b = (0.1 * torch.randn(3 * c, device=dev, generator=g)).bfloat16().requires_grad_()
    wo = (torch.randn(c, c, device=dev, generator=g) / c**0.5).bfloat16()
    o = torch.randn(bsz, heads, n, c // heads, device=dev, generator=g).bfloat16()
    gy = torch.randn(3, bsz, heads, n, c // heads, device=dev, generator=g).bfloat16()
    for _ in range(reps):
        ja.core_forward(q, k, v, d**-0.5)
        ja.core_backward(dout, q, k, v, out, lse, d**-0.5)
        y = jp.qkv_projection(x, w, b, heads)
        torch.autograd.grad(y, (x, w, b), gy)
        jp.heads_projection(o, wo, None)
    torch.cuda.synchronize()
    print("profile_kernels: done", file=sys.stderr)


def swin_block(reps: int = 5) -> None:
    from jigsaw_amd import swin as js
    from jigsaw_amd.conv import TileGroup

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(2)

    slabs = {}

    def comm(data, buffer, direction, *, group, async_op):
        key = (tuple(buffer.shape), direction, id(group))
        if key not in slabs:  # the neighbour's slab: a seeded stand-in, made once per slab shape
            slabs[key] = torch.randn(buffer.shape, device=dev, generator=g).to(buffer.dtype)
        return slabs[key], None

    n, dim = (256, 256), 128
    block = js.SwinBlock(dim, 4, 8, n, (TileGroup(2, 0), TileGroup(2, 1)), comm, shift=4, device=dev)
    x = torch.randn(1, *n, dim, device=dev, generator=g).bfloat16().requires_grad_()
    gout = torch.randn(1, *n, dim, device=dev, generator=g).bfloat16()
    leaves = [x, *block.parameters()]
    for _ in range(reps):
        for t in leaves:
            t.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = block(x)
        y.backward(gout)
    torch.cuda.synchronize()
    print("profile_kernels: done", file=sys.stderr)


def attention_fp32(reps: int = 3) -> None:
    from jigsaw_amd import attention as ja

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(4)
    for d in (64, 128, 32):
        b, h, n = 1, 8, 4096
        q, k, v, dout = (torch.randn(b, h, n, d, device=dev, generator=g) / 8 for _ in range(4))
        scale = d**-0.5
        for _ in range(reps):
            out, lse = ja.core_forward(q, k, v, scale)
            ja.core_backward(dout, q, k, v, out, lse, scale)
        torch.cuda.synchronize()
    print("profile_kernels: done", file=sys.stderr)


def sharded_layernorm(reps: int = 3) -> None:
    from jigsaw_amd import layernorm as jl

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(3)
    for rows, cols in ((1 << 18, 256), (1 << 20, 64), (1 << 18, 132)):
        x = torch.randn(rows, cols, device=dev, generator=g).bfloat16().requires_grad_()
        w = torch.ones(cols, device=dev, dtype=torch.bfloat16, requires_grad=True)
        b = torch.zeros(cols, device=dev, dtype=torch.bfloat16, requires_grad=True)
        gout = torch.randn(rows, cols, device=dev, generator=g).bfloat16()
        for _ in range(reps):
            x.grad = w.grad = b.grad = None
            jl.layer_norm(x, w, b, None).backward(gout)
        torch.cuda.synchronize()
    print("profile_kernels: done", file=sys.stderr)


if __name__ == "__main__":
    if sys.argv[1:] == ["around-attention"]:
        around_attention()
    elif sys.argv[1:] == ["sharded-layernorm"]:
        sharded_layernorm()
    elif sys.argv[1:] == ["attention-fp32"]:
        attention_fp32()
    elif sys.argv[1:] == ["swin-block"]:
        swin_block()
    elif sys.argv[1:]:
        raise SystemExit(f"unknown argument {sys.argv[1:]}; known: 'around-attention', 'swin-block', 'sharded-layernorm', 'attention-fp32'")
    else:
        main()
