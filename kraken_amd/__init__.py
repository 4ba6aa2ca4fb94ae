"""MI355X-native table engine behind Kraken's parameter-server Table/Optim/Initializer
interfaces. The compute lives in libkraken_hip.so (HIP, gfx950); this package is the thin
host-side mirror of the reference's interface used by tests and benchmarks."""
from .api import (ASYNC, DEVICE_PTRS, DenseBag, DenseTable, DeviceArray, Event, Initializer,  # noqa: F401
                  InitializerType, KrakenHipError, Optim, OptimType, SparseTable, StateType, TableGroup,
                  coo_to_dense, dedup, lib, synchronize)
