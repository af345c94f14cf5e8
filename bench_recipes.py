"""Times the training recipes' products on synthetic operands of a model's expert shapes: for the blockwise FP8, MXFP8
and NVFP4 recipes and for plain bf16 matrices, the forward product, the input's gradient and the matrices' gradient
(each with the passes that quantize or transpose its operands timed beside it). One JSON line a product.

    python bench_recipes.py [--shape mixtral|deepseek] [--steps 5]

`tflops` counts 2 x rows x depth x width for the product alone; `prepare_us` is the operands' quantizing / transposing
passes of that product (the matrices' own quantization, done once a step for all three products, is not timed)."""

import argparse
import json

import torch

from dew_amd import formats, gemm, ops, projections

SHAPES = {
    # groups, rows a group, depth, width: the gate/up and the down projection of each model's experts
    "mixtral": [(8, 4096, 4096, 14336), (8, 4096, 14336, 4096)],
    "deepseek": [(32, 1024, 7168, 2048), (32, 1024, 2048, 7168)],
}


def timed(call, steps: int) -> float:
    """Microseconds a call, from events on the stream the kernels are launched on (torch's current one)."""
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    call()
    start.record()
    for _ in range(steps):
        call()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps * 1e3


def products(recipe: str, x, w, dy, blocks, offsets):
    """(name, prepare call, product call) for the recipe's three products, operands prepared once outside the timing."""
    sizes = offsets[1:] - offsets[:-1]
    if recipe == "bf16":
        bank, bank_t = ops.prepare(formats.Bf16(w)), ops.prepare(formats.Bf16(w).T)
        rows_t, _ = ops.transpose_columns(x, as_bank=False)
        dy_bank, _ = ops.transpose_columns(dy, as_bank=True)
        return [("forward", None, lambda: ops.grouped_gemm(x, bank, offsets)),
                ("d_x", None, lambda: ops.grouped_gemm(dy, bank_t, offsets)),
                ("d_w", lambda: (ops.transpose_columns(x, as_bank=False), ops.transpose_columns(dy, as_bank=True)),
                 lambda: ops.kernel_gradient_bf16(rows_t, dy_bank, offsets))]
    if recipe == "nvfp4":
        bank, bank_t = projections.nvfp4_matrices(w), projections.nvfp4_matrices(w.transpose(1, 2).contiguous())
        rows, cotangents = projections.nvfp4_rows(x), projections.nvfp4_rows(dy)
        rows_t, rows_scale = ops.transpose_columns(x, nvfp4=True, as_bank=False)
        dy_bank, dy_scale = ops.transpose_columns(dy, nvfp4=True, as_bank=True)
        return [("forward", lambda: projections.nvfp4_rows(x), lambda: projections.nvfp4_block_product(rows, bank, sizes)),
                ("d_x", lambda: projections.nvfp4_rows(dy), lambda: projections.nvfp4_block_product(cotangents, bank_t, sizes)),
                ("d_w", lambda: (ops.transpose_columns(x, nvfp4=True, as_bank=False), ops.transpose_columns(dy, nvfp4=True, as_bank=True)),
                 lambda: ops.kernel_gradient_bf16(rows_t, dy_bank, offsets, lhs_scale=rows_scale, rhs_scale=dy_scale))]
    mx = recipe == "mxfp8"
    if mx:
        bank, bank_t = gemm.prepared(formats.MxFp8.quantized(w)), gemm.prepared(formats.MxFp8.quantized(w.transpose(1, 2).contiguous()))
        quantized, product = projections.mxfp8_rows, projections.mxfp8_product
    else:
        bank, bank_t = gemm.prepared(projections.blocks_quantized(w)), gemm.prepared(projections.blocks_quantized(w.transpose(1, 2).contiguous()))
        quantized, product = projections.rows_quantized, projections.blockwise_fp8_product
    rows, cotangents = quantized(x), quantized(dy)
    codes, scales = ops.quantize_columns(x, mx=mx, as_bank=False)
    dy_bank = ops.quantize_columns(dy, mx=mx, as_bank=True)
    return [("forward", lambda: quantized(x), lambda: product(rows, bank, sizes)),
            ("d_x", lambda: quantized(dy), lambda: product(cotangents, bank_t, sizes)),
            ("d_w", lambda: (ops.quantize_columns(x, mx=mx, as_bank=False), ops.quantize_columns(dy, mx=mx, as_bank=True)),
             lambda: ops.kernel_gradient_mxfp8(codes, scales, dy_bank, offsets))]


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--shape", default="mixtral", choices=sorted(SHAPES))
    parser.add_argument("--steps", type=int, default=5)
    parser.add_argument("--recipes", default="blockwise_fp8,mxfp8,nvfp4,bf16")
    args = parser.parse_args()
    ops.device_check()
    device = torch.device("cuda:0")
    for groups, each, depth, width in SHAPES[args.shape]:
        generator = torch.Generator(device=device).manual_seed(0)
        tokens = groups * each
        x = torch.randn((tokens, depth), device=device, generator=generator).to(torch.bfloat16)
        dy = torch.randn((tokens, width), device=device, generator=generator).to(torch.bfloat16)
        w = (torch.randn((groups, depth, width), device=device, generator=generator) * 0.02).to(torch.bfloat16)
        offsets = torch.arange(0, tokens + 1, each, dtype=torch.int32, device=device)
        for recipe in args.recipes.split(","):
            for name, prepare, product in products(recipe, x, w, dy, [each // 128] * groups, offsets):
                spent = timed(product, args.steps)
                print(json.dumps({"recipe": recipe, "product": name, "groups": groups, "rows_a_group": each, "depth": depth, "width": width,
                                  "us": round(spent, 1), "tflops": round(2.0 * tokens * depth * width / spent / 1e6, 1),
                                  "prepare_us": None if prepare is None else round(timed(prepare, args.steps), 1), "data": "synthetic"}),
                      flush=True)


if __name__ == "__main__":
    main()
