"""MI355X-native device backend for gguf-trainer's training hot path.

Layout:
  csrc/           hand-written HIP kernels for gfx950 and the C ABI (include/ggufhip.h)
  lib.py          ctypes binding of libggufhip.so; raises when the library is missing
  autograd.py     host tape: Tensor, backward, checkpoint, LoRA-aware linear, validators, dispatch
                  (mirror of src/model/autograd.ts above the OpsBackend boundary; no CPU ops)
  hip_backend.py  HipBackend: OpsBackend + RegionBackend + the buffer surface of WebGPUBackend
  optim.py        AdamWHip / MuonHip (mirrors of AdamWGpu / MuonGpu)
  arch.py         llama / qwen3 / gemma3 forward graphs (op order of src/arch/*.ts)
  train.py        the device-resident step loop (src/backend/train-gpu.ts:162-258)
"""
