"""TEST INFRASTRUCTURE ONLY.

CPU restatement of the algorithm on the graded path, used as the checker by `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py`.  Nothing in the
product package (`flex_rnn_amd/`) imports, calls or falls back to anything here.

  recurrence.py  per-timestep loop restating /root/reference/flex_rnn/jit.py:23-36 and
                 README.md:28-38, written independently of the package's `jit.naive`,
                 plus closed forms / invariants that pin it.
  plan_exec.py   executes the partitioned plan (fw / reverse scan / gradient pass with
                 checkpoints, saved row-sums and row-axis accumulation) with torch ops on
                 the CPU; this pins the graph partition against autograd of the loop.

Parity status: every function here is pinned by closed forms, brute force on tiny
inputs or `torch.autograd`; see the header of each file.  The reference ships no
golden vectors for this path (its only test is a GPU script), and its Python was
not imported.
"""
