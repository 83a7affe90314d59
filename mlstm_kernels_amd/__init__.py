"""mlstm_kernels_amd: the mLSTM hot path (TFLA chunkwise forward/backward, fused recurrent decode step)
as hand-written gfx950 HIP kernels behind a C ABI, exposed through the operator interface of
NX-AI/mlstm_kernels (``mLSTMBackend``, ``get_mlstm_kernel('chunkwise--hip_xl_chunk')``, step kernel
``'hip'``).  There is no CPU or PyTorch fallback: every kernel call raises if libmlstm_hip.so is missing."""

__version__ = "0.1.0"
