"""CPU parity oracle for the LoRA training step (test infrastructure only).

`oracle.cpu` wraps the C++ restatement of the reference's kernels;
`oracle.reference_step` restates the reference's model, loss, backward and
optimizer step on top of those kernels. Only tests, the smoke check and the
benchmark's cpu_baseline leg import this package.
"""
