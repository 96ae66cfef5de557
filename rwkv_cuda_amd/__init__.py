"""rwkv_cuda_amd: the WKV recurrence family and depthwise_conv1d of BlinkDL/RWKV-CUDA as
hand-written HIP kernels for MI355X (gfx950), behind a C ABI (include/rwkv_hip.h) and the
reference's own torch.autograd.Function interface.

    wkv               WKV.apply(B,T,C,w,u,k,v)                       RWKV-4, fp32
    depthwise_conv1d  TimeX.apply(w,k,B,C,T,eps)                     fp32
    wkv5_bf16         WKV_5.apply(B,T,C,H,r,k,v,w,u)                 bf16
    wkv5              WKV_5.apply(B,T,C,H,r,k,v,w,u)                 fp32
    wkv5a             WKV_5A.apply(r,k,v,w1,u1,w2,u2)                fp32, two-sided decay and bonus
    wkv6              WKV_6.apply(B,T,C,H,r,k,v,w,u)                 bf16
    wkv6_state        WKV_6STATE.apply(B,T,C,H,r,k,v,w,u,s)          bf16
    rwkv7_fast_fused  RWKV7_STATE_PASSING_CLAMPW_CUDA(s0,r,w,k,v,a,b) -> (y, sT)

There is no CPU or eager fallback: the ops need the compiled library and a HIP device.
"""

from . import _lib  # noqa: F401
