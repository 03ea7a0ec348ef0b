"""MI355X-native MoE FFN layer of Titanic Flash: C-ABI kernel library, C++ host mirror of the reference's Rust
operators, and the python helpers the tests and the benchmark drive them with."""
from . import contracts, host, native, synth  # noqa: F401
