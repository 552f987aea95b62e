"""Autocast policy of the operators.

The reference wraps its GEMM-type Functions in custom_fwd(cast_inputs=float16)
and its LayerNorm / loss Functions in custom_fwd(cast_inputs=float32)
(cubework/module/parallel_2d/_operation.py:17,96,176,255,309,363;
cubework/module/loss/loss_1d.py:13). The MI355X kernels take bf16 and fp32,
so inside an autocast region GEMM-type operators cast to bfloat16; outside
autocast nothing is cast, as in the reference.
"""
import functools

import torch

gemm_fwd = functools.partial(torch.amp.custom_fwd, device_type="cuda", cast_inputs=torch.bfloat16)
fp32_fwd = functools.partial(torch.amp.custom_fwd, device_type="cuda", cast_inputs=torch.float32)
bwd = functools.partial(torch.amp.custom_bwd, device_type="cuda")
