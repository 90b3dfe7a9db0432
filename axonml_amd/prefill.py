"""Prefill-path benchmark helper: quantized GEMM with bf16 and f32 activations at the 7B model's projection shapes."""
import ctypes as C

import numpy as np

from ._lib import MEM_DEVICE
from .quant import QuantType, f32_to_bf16_bits

MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16/bf16, published


BLK32_TYPES = (QuantType.Q4_0, QuantType.Q4_1, QuantType.Q5_0, QuantType.Q5_1, QuantType.Q8_0)


def bench(ctx, log=print, ms=(128, 512, 2048), ns=(4096, 14336), k=4096, types=(QuantType.Q4_K, QuantType.Q5_K, QuantType.Q5_1), iters=20,
          f32_rows=True):
    """Times axq_gemm_bf16 (and, with f32_rows, the same product from f32 rows through axq_gemv_f32) per shape and type."""
    lib = ctx.lib
    rng = np.random.default_rng(0)
    out = []
    for qt in types:
        for n in ns:
            f = ctx.malloc(n * k * 4)
            ctx.check(lib.axq_fill_normal_f32(ctx.handle, f, n * k, 0.0, 0.02, 0.0, 0.0, 77))
            h = C.c_void_p()
            ctx.check(lib.axq_weight_quantize(ctx.handle, int(qt), n, k, f, MEM_DEVICE, C.byref(h)))
            ctx.free(f)
            for m in ms:
                x = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
                xd = ctx.to_device(x)
                yd = ctx.malloc(m * n * 4)
                for _ in range(3):
                    ctx.check(lib.axq_gemm_bf16(ctx.handle, h, xd, m, yd, MEM_DEVICE))
                ctx.synchronize()
                ctx.timer_start()
                for _ in range(iters):
                    ctx.check(lib.axq_gemm_bf16(ctx.handle, h, xd, m, yd, MEM_DEVICE))
                t = ctx.timer_stop() / iters
                flops = 2.0 * m * n * k
                r = {"type": str(qt), "m": m, "n": n, "k": k, "ms": t, "tflops": flops / (t * 1e-3) / 1e12,
                     "route": "hand-written MFMA GEMM, centred scaled codes as f16, one product per weight" if qt in (QuantType.Q4_K, QuantType.Q5_K)
                     else "hand-written MFMA GEMM, centred codes as f16, one product per weight, block scales by the vector ALU"
                     if k % 256 == 0 and qt in BLK32_TYPES
                     else "hand-written MFMA GEMM, weights dequantised to two f16 terms, two products per weight"}
                r["frac_of_mfma_f16_peak"] = r["tflops"] / MFMA_F16_PEAK_TFLOPS
                out.append(r)
                log(f"  prefill {r['type']} M={m} N={n}: {t * 1e3:.1f} us, {r['tflops']:.1f} TFLOP/s")
                ctx.free(xd)
                if not f32_rows:
                    ctx.free(yd)
                    continue
                # the same product from f32 rows (axq_gemv_f32 sends 40 rows or more through the GEMM as two f16 rows each)
                xf = ctx.to_device(rng.standard_normal((m, k)).astype(np.float32))
                for _ in range(3):
                    ctx.check(lib.axq_gemv_f32(ctx.handle, h, xf, m, None, yd, MEM_DEVICE))
                ctx.synchronize()
                ctx.timer_start()
                for _ in range(iters):
                    ctx.check(lib.axq_gemv_f32(ctx.handle, h, xf, m, None, yd, MEM_DEVICE))
                t32 = ctx.timer_stop() / iters
                r["f32_rows_ms"], r["f32_rows_tflops"] = t32, flops / (t32 * 1e-3) / 1e12
                log(f"          f32 rows      : {t32 * 1e3:.1f} us, {r['f32_rows_tflops']:.1f} TFLOP/s of useful work")
                ctx.free(xf)
                ctx.free(yd)
            lib.axq_weight_free(ctx.handle, h)
    return out
