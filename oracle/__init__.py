"""TEST INFRASTRUCTURE: CPU oracle for the mapped-convolution hot path.

Only tests, `__graft_entry__.smoke()` and the benchmark's CPU-baseline leg may
import this package.  `oracle.ops` exposes the C restatement under the same op
names and argument order as the shipped `_C` boundary, on CPU tensors;
`oracle.reference` loads the reference's own CPU build from oracle/_ref when it
has been built.
"""
