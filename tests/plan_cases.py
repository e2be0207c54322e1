"""The calls whose kernel routing is pinned: every bench.py workload (the BASELINE
configs among them), as (entry point, dtype, sizes in the entry point's order, layout)."""


def _ln(n, c, dt, backward=True):
    out = [("layer_norm", dt, (n, c), "NCHW")]
    if backward:
        out.append(("layer_norm_grad", dt, (n, c), "NCHW"))
    return out


def _rows(fwd, bwd, n, c, dt):
    return [(fwd, dt, (n, 1, c), "NCHW"), (bwd, dt, (n, 1, c), "NCHW")]


def _bn(n, c, s, dt, layout="NCHW"):
    return [("batch_norm_training_forward", dt, (n, c, s), layout),
            ("batch_norm_training_backward", dt, (n, c, s), layout)]


def _gn(n, g, d, s, dt, layout="NCHW"):
    return [("group_norm_forward", dt, (n, g, d, s), layout),
            ("group_norm_grad", dt, (n, g, d, s), layout)]


CASES = {
    # BASELINE configs
    "softmax_f16_16x32x512x512": _rows("softmax", "softmax_grad", 16 * 32 * 512, 512, "float16"),
    "layer_norm_f32_8192x1024_fwd": _ln(8192, 1024, "float32", backward=False),
    "batch_norm_f32_64x256x56x56": _bn(64, 256, 56 * 56, "float32"),
    "group_norm_bf16_32x512x64x64_g32": _gn(32, 32, 16, 64 * 64, "bfloat16"),
    "layer_norm_bf16_8192x12288": _ln(8192, 12288, "bfloat16"),
    "layer_norm_bf16_65536x1000": _ln(65536, 1000, "bfloat16"),
    # the rest of the bench sweep
    "layer_norm_bf16_8192x4096": _ln(8192, 4096, "bfloat16"),
    "layer_norm_f32_8192x4096": _ln(8192, 4096, "float32"),
    "layer_norm_bf16_32768x4096": _ln(32768, 4096, "bfloat16"),
    "layer_norm_bf16_32768x12288": _ln(32768, 12288, "bfloat16"),
    "softmax_f16_8192x4096": _rows("softmax", "softmax_grad", 8192, 4096, "float16"),
    "softmax_f32_8192x4096": _rows("softmax", "softmax_grad", 8192, 4096, "float32"),
    "softmax_cross_entropy_f32_8192x4096": _rows("softmax_cross_entropy_loss_forward",
                                                 "softmax_cross_entropy_loss_backward", 8192, 4096,
                                                 "float32"),
    "l2_norm_bf16_8192x4096": _rows("l2_norm", "l2_norm_grad", 8192, 4096, "bfloat16"),
    "l2_norm_f32_8192x4096": _rows("l2_norm", "l2_norm_grad", 8192, 4096, "float32"),
    "softmax_bf16_605184x197": _rows("softmax", "softmax_grad", 605184, 197, "bfloat16"),
    "layer_norm_bf16_1048576x64": _ln(1048576, 64, "bfloat16"),
    "softmax_f32_2048x128256": _rows("softmax", "softmax_grad", 2048, 128256, "float32"),
    "batch_norm_f32_64x256x57x57": _bn(64, 256, 57 * 57, "float32"),
    "softmax_bf16_4096x50257": _rows("softmax", "softmax_grad", 4096, 50257, "bfloat16"),
    "group_norm_bf16_32x64x64x512_g32_nhwc": _gn(32, 32, 16, 64 * 64, "bfloat16", "NHWC"),
}
