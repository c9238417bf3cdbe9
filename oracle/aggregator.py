"""TEST INFRASTRUCTURE -- CPU oracle of the aggregation pipeline of one rank.

numpy restatement of self_benchmark/a64fx/model/layers/aggregator.py: forward :16-119,
backward :121-208, on CSR tuples (rowptr, col, value, (rows, cols)) and with the
boundary all-to-all replaced by buffers the caller moves between simulated ranks.

Pinning: the reference holds no test for the aggregator.  What fixes these functions
is (a) they only compose oracle.spmm (pinned in tests/test_oracle_spmm.py) and (b) the
all-ranks invariant of tests/test_pipeline_invariant.py: with every rank simulated in
one process, ``A_local X + A_from exchange(A_to X)`` must equal the plain global
product ``A X`` on every rank, and likewise for the transposed (gradient) direction.
"""
import numpy as np

from . import quantization as oquant
from . import spmm as ospmm


def _mm(mat, x, out):
    rowptr, col, val, _ = mat
    return ospmm.spmm(rowptr, col, val, x, out)


def _mm_t(mat, g, out):
    rowptr, col, val, shape = mat
    return ospmm.spmm_transposed(rowptr, col, val, g, out, shape[1])


def forward_send(a_to, x):
    """aggregator.py:44-49: send_buf = 0; send_buf += A_to @ X (pre-aggregation)."""
    send = np.zeros((a_to[3][0], x.shape[1]), dtype=np.float32)
    return _mm(a_to, x, send)


def forward_send_raw(idx_nodes_send_to_others, x):
    """aggregator.py:51: send_buf = X[idx]."""
    return np.ascontiguousarray(x[np.asarray(idx_nodes_send_to_others, dtype=np.int64)])


def forward_out(local_adj, a_from_or_remote, x, recv_buf):
    """aggregator.py:67-70, :100-104: out = 0; out += A_local @ X; out += A_from @ recv."""
    out = np.zeros((local_adj[3][0], x.shape[1]), dtype=np.float32)
    _mm(local_adj, x, out)
    if recv_buf is not None and recv_buf.shape[0] != 0:
        _mm(a_from_or_remote, recv_buf, out)
    return out


def backward_recv(a_from_or_remote, grad):
    """aggregator.py:144-149: recv_buf = 0; recv_buf += A_from^T @ G (outgoing halo grads)."""
    out = np.zeros((a_from_or_remote[3][1], grad.shape[1]), dtype=np.float32)
    return _mm_t(a_from_or_remote, grad, out)


def backward_out(local_adj, a_to, grad, send_buf_in):
    """aggregator.py:167-170, :192-195: dX = 0; dX += A_local^T @ G; dX += A_to^T @ send_buf."""
    dx = np.zeros((local_adj[3][1], grad.shape[1]), dtype=np.float32)
    _mm_t(local_adj, grad, dx)
    if send_buf_in is not None and send_buf_in.shape[0] != 0:
        _mm_t(a_to, send_buf_in, dx)
    return dx


def backward_out_raw(local_adj, idx_nodes_send_to_others, grad, send_buf_in):
    """aggregator.py:197-199: dX.index_add_(0, idx, send_buf), rows added in index order."""
    dx = np.zeros((local_adj[3][1], grad.shape[1]), dtype=np.float32)
    _mm_t(local_adj, grad, dx)
    for i, r in enumerate(np.asarray(idx_nodes_send_to_others, dtype=np.int64)):
        dx[r] += send_buf_in[i]
    return dx


def quantized_wire(outgoing, splits, bits):
    """What the peers see of an outgoing boundary buffer in a quantised exchange
    (communicator.py:281-311, aggregator.py:83-88): every peer's segment packed on its own,
    parameters rounded through bf16 on the wire, dequantised with those.  Row i of the result
    is what the owner of row i's segment receives for it."""
    if outgoing.shape[0] == 0:
        return outgoing.copy()
    packed, params = oquant.quantize_segments(outgoing, splits, bits)
    return oquant.dequantize_segments(packed, oquant.params_over_the_wire(params), splits, bits)
