"""MI355X-native MoE dispatch / combine behind the operator API of pplx-garden.

Layout mirrors the part of the reference's `pplx_garden` package that this
path touches: `kernels` (the operator), `native` (the binding to the compiled
library), `distributed` (the group object an operator is built on) and `utils`.
"""

__version__ = "0.1"
