"""The hand-written gfx950 kernels: build (:mod:`build`), load (:mod:`lib`), call (:mod:`ops`)."""
