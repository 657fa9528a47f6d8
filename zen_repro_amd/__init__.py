"""MI355X-native sparse-gradient select / hash-partition / merge path of ZEN,
behind the reference's Python call surface (extensions.cuda.functions,
tensor_load_balance.TensorPartition, comm.LoadBalanceAllreduce, train.compress).
All compute runs in hand-written HIP kernels reached through libzen_hip.so."""
from .functions import hash_index, last_status, sparse_balance  # noqa: F401
from .tensor_load_balance import TensorPartition  # noqa: F401
from .comm import LoadBalanceAllreduce, LocalGroup  # noqa: F401
from .compress import compress, compress_with_allgather, topk_threshold  # noqa: F401
from .hook import SparseCommHook  # noqa: F401
