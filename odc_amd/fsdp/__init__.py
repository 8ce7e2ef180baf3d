"""Minibatch hooks and call-site glue for torch FSDP1 / FSDP2 on top of the primitives."""
