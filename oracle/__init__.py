"""CPU oracle for the helium MI355X backend — TEST INFRASTRUCTURE ONLY.

A plain numpy / C restatement of the reference's semantics for the hot path, used as the checker by `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py`. Nothing in `helium_amd/` may import it and
no product path may route through it.

The reference (Rust + NVRTC-compiled CUDA) cannot be built or run here and has no CPU execution path of its
own (`Device::Cpu` is `todo!()`, helium/src/raw_tensor.rs:100,1073), so every function below restates the
reference source it cites and is pinned by the vectors the reference's own tests hold
(tests/golden/tensor_ops.json and tests/golden/autodiff.json, transcribed from helium/tests/tensor_ops.rs,
helium/tests/autodiff.rs, helium/tests/loss.rs and the unit tests inside the reference's source files) plus closed
forms / brute force where those leave gaps. The pins themselves are tests/test_oracle_cpu.py (convolution and its
gradients, the autodiff / loss / matmul vectors, Compare / Select / casts, scalar functions, reductions, the fusion
IR and the README graph's closed forms), tests/test_pointwise_cpu.py (the pointwise known answers of tensor_ops.rs),
tests/test_permute_cpu.py (permute vectors, numpy.transpose, a brute-force walk) and tests/test_plan_cpu.py
(hand-derived plans).

Parity status per module is stated in each module's docstring; anything not pinned says "parity unpinned".
"""
