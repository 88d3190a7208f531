"""CPU oracle for the helium MI355X backend — TEST INFRASTRUCTURE ONLY.

A plain numpy / C restatement of the reference's semantics for the hot path, used as the checker by `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py`. Nothing in `helium_amd/` may import it and
no product path may route through it.

The reference (Rust + NVRTC-compiled CUDA) cannot be built or run here and has no CPU execution path of its
own (`Device::Cpu` is `todo!()`, helium/src/raw_tensor.rs:100,1073), so every function below restates the
reference source it cites and is pinned by the vectors the reference's own tests hold
(tests/golden/*.json, transcribed from helium/tests/tensor_ops.rs, helium/tests/autodiff.rs and the unit tests
inside the reference's source files) plus closed forms / brute force where those leave gaps.

Parity status per module is stated in each module's docstring; anything not pinned says "parity unpinned".
"""
