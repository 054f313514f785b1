"""MI355X (gfx950) kernel backend for the FrankenTorch transformer forward op set.

    kernel_hip   the `ft_kernel_cpu` operator surface (host arrays in, host array out)
    device       device-pointer kernels, buffers, streams, events
    fused        resident tensors, Batch, EncoderHip, Gpt2Hip (the `ft_kernel_metal::fused` shape)
    core         TensorMeta / DType / Device / KernelError / HipError
    synth        seeded synthetic inputs for the benchmark configurations

Everything computes in hand-written HIP kernels loaded from libft_kernel_hip.so; there is no CPU
fallback. Importing the package does not touch the GPU.
"""

__all__ = ["kernel_hip", "device", "fused", "core", "synth"]
