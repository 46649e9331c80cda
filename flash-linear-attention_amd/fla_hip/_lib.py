"""ctypes binding of libgdn_hip.so (declarations follow include/gdn_hip.h)."""
from __future__ import annotations

import ctypes
import os
import threading
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint32, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get('FLA_HIP_LIBRARY') or os.path.join(_HERE, '_C', 'libgdn_hip.so')

ABI_VERSION = 13

GDN_OK = 0
GDN_ERR_INVALID = -1
GDN_ERR_UNSUPPORTED = -2
GDN_ERR_LAUNCH = -3
GDN_ERR_WORKSPACE = -4

DTYPE_BF16, DTYPE_F16, DTYPE_F32 = 0, 1, 2

FLAG_QK_L2NORM = 1 << 0
FLAG_BETA_SIGMOID = 1 << 1
FLAG_NEG_EIGVAL = 1 << 2
FLAG_STATE_V_FIRST = 1 << 3
FLAG_BETA_VECTOR = 1 << 4
FLAG_CU_INT32 = 1 << 5
FLAG_SLOT_INT32 = 1 << 6
FLAG_SLOT_PER_TOKEN = 1 << 7
FLAG_STATE_PER_TOKEN = 1 << 8
FLAG_STATE_BF16 = 1 << 9
FLAG_SCAN_WIDE = 1 << 17
FLAG_SCAN_SEGMENTS = 1 << 18
FLAG_SEQ_ORDER = 1 << 19
FLAG_SCAN_NO_PAIR = 1 << 20
FLAG_SCAN_PAIR = 1 << 21
FLAG_SCAN_NO_WARM = 1 << 22
FLAG_RECORD_P = 1 << 23

ACT_NONE, ACT_SILU, ACT_SIGMOID = 0, 1, 2

# name -> (restype, argtypes); one entry per declaration in include/gdn_hip.h
SIGNATURES = {
    'gdn_hip_abi_version': (c_int, []),
    'gdn_last_error': (c_char_p, []),
    'gdn_fused_recurrent_fwd': (c_int, [
        c_void_p, c_void_p, c_void_p,                      # q k v
        c_void_p, c_void_p, c_void_p, c_void_p,            # g beta gk gv
        c_void_p, c_void_p,                                # A_log dt_bias
        c_void_p, c_void_p, c_void_p,                      # h0 ht o
        c_void_p, c_void_p, c_void_p, c_int64,             # cu_seqlens state_slots num_accepted slots_stride
        c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T H HV K V N
        c_float, c_int, c_int, c_uint32, c_void_p]),
    'gdn_fused_recurrent_kda_fwd': (c_int, [
        c_void_p, c_void_p, c_void_p,                      # q k v
        c_void_p, c_void_p,                                # g beta
        c_void_p, c_void_p, c_float, c_int,                # A_log dt_bias lower_bound gate_mode
        c_void_p, c_void_p, c_void_p,                      # h0 ht o
        c_void_p, c_void_p, c_void_p, c_int64,             # cu_seqlens state_slots num_accepted slots_stride
        c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T H HV K V N
        c_float, c_int, c_int, c_uint32, c_void_p]),
    'gdn_fused_recurrent_comba_fwd': (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p,            # q k p v
        c_void_p, c_void_p,                                # g beta
        c_void_p, c_void_p, c_void_p,                      # h0 ht o
        c_void_p,                                          # cu_seqlens
        c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T H HV K V N
        c_float, c_int, c_int, c_uint32, c_void_p]),
    'gdn_chunk_workspace_bytes': (c_size_t, [c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_uint32]),
    'gdn_causal_conv1d_fwd': (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,  # x weight bias residual initial_state
        c_void_p, c_void_p, c_void_p,                      # y final_state cu_seqlens
        c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T D W N stride_x_n stride_x_t
        c_int, c_int, c_int, c_int, c_uint32, c_void_p]),  # x_dtype w_dtype state_dtype activation flags stream
    'gdn_causal_conv1d_update': (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,      # x cache residual weight bias y
        c_int64, c_int64, c_int64, c_int64, c_int64,       # N D W stride_x_n stride_y_n
        c_int, c_int, c_int, c_int, c_void_p]),            # x_dtype w_dtype cache_dtype activation stream
    'gdn_norm_gated_fwd': (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,  # x g weight bias residual
        c_void_p, c_void_p, c_void_p, c_void_p,            # y residual_out mean rstd
        c_int64, c_int64, c_float,                         # T D eps
        c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),   # x/w/res/res_out dtype, activation, is_rms_norm, stream
}
_CHUNK_ARGS = [
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,      # q k v g beta
    c_void_p, c_void_p,                                    # A_log dt_bias
    c_void_p, c_void_p, c_void_p,                          # h0 ht o
    c_void_p, c_void_p, c_void_p,                          # cu_seqlens chunk_table chunk_offsets
    c_void_p, c_size_t,                                    # workspace, bytes
    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,  # B T H HV K V
    c_int64, c_int64,                                      # N num_chunks
    c_float, c_int, c_int, c_uint32, c_void_p]
for _name in ('gdn_chunk_fwd', 'gdn_chunk_fwd_prepare', 'gdn_chunk_fwd_scan'):
    SIGNATURES[_name] = (c_int, _CHUNK_ARGS)

SIGNATURES['gdn_chunk_fwd_static'] = (c_int, _CHUNK_ARGS[:13] + _CHUNK_ARGS[15:])     # no workspace, no size
SIGNATURES['gdn_chunk_bwd_workspace_bytes'] = (c_size_t, [c_int64, c_int64, c_int64])
SIGNATURES['gdn_chunk_bwd'] = (c_int, [
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,  # q k v g beta
    c_void_p, c_void_p, c_void_p,                      # h0 dout dht
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,      # dq dk dv dg dbeta dh0
    c_void_p, c_void_p, c_void_p,                      # cu_seqlens chunk_table chunk_offsets
    c_void_p, c_size_t,                                # workspace workspace_bytes
    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T H HV K V N num_chunks
    c_float, c_int, c_int, c_uint32, c_void_p])
SIGNATURES['gdn_chunk_bwd_qk_l2norm_workspace_bytes'] = (c_size_t, [c_int64, c_int64, c_int64, c_int64])
SIGNATURES['gdn_chunk_bwd_qk_l2norm'] = SIGNATURES['gdn_chunk_bwd']      # (q, k before their l2 normalisation)
SIGNATURES['gdn_chunk_comba_bwd'] = (c_int, [
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,  # q k p v g beta
    c_void_p, c_void_p, c_void_p,                      # h0 dout dht
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,      # dq dk dp dv dg dbeta dh0
    c_void_p, c_void_p, c_void_p,                      # cu_seqlens chunk_table chunk_offsets
    c_void_p, c_size_t,                                # workspace workspace_bytes
    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T H HV K V N num_chunks
    c_float, c_int, c_int, c_uint32, c_void_p])
SIGNATURES['gdn_chunk_comba_bwd_qk_l2norm_workspace_bytes'] = (c_size_t, [c_int64, c_int64, c_int64])
SIGNATURES['gdn_chunk_comba_bwd_qk_l2norm'] = SIGNATURES['gdn_chunk_comba_bwd']      # (q, k, p before their l2 normalisation)
SIGNATURES['gdn_chunk_kda_bwd_workspace_bytes'] = (c_size_t, [c_int64, c_int64])
SIGNATURES['gdn_chunk_kda_bwd'] = SIGNATURES['gdn_chunk_bwd']        # (g: [B,T,HV,K] fp32, dg likewise)
SIGNATURES['gdn_l2norm_fwd'] = (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p])
SIGNATURES['gdn_l2norm_bwd'] = (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p])
SIGNATURES['gdn_fused_recurrent_delta_bwd_value_block'] = (c_int64, [c_int64])
SIGNATURES['gdn_fused_recurrent_delta_bwd'] = (c_int, [
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,      # q k v beta dout h0 dht
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,      # dq_part dk_part dv db dh0 u_workspace cu_seqlens
    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,                      # B T H K V N
    c_float, c_int, c_int, c_uint32, c_void_p])
SIGNATURES['gdn_chunk_kda_workspace_bytes'] = (c_size_t, [c_int64, c_int64])
SIGNATURES['gdn_chunk_kda_fwd'] = (c_int, [
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,  # q k v g beta
    c_void_p, c_void_p, c_float, c_int,                # A_log dt_bias lower_bound gate_mode
    c_void_p, c_void_p, c_void_p,                      # h0 ht o
    c_void_p, c_void_p, c_void_p,                      # cu_seqlens chunk_table chunk_offsets
    c_void_p, c_size_t,                                # workspace workspace_bytes
    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T H HV K V N num_chunks
    c_float, c_int, c_int, c_uint32, c_void_p])
SIGNATURES['gdn_chunk_kda_fwd_states'] = (c_int, SIGNATURES['gdn_chunk_kda_fwd'][1][:12] + [c_void_p] + SIGNATURES['gdn_chunk_kda_fwd'][1][12:])
SIGNATURES['gdn_chunk_comba_fwd'] = (c_int, [
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # q k v p g beta
    c_void_p, c_void_p, c_void_p,                      # h0 ht o
    c_void_p, c_void_p, c_void_p,                      # cu_seqlens chunk_table chunk_offsets
    c_void_p, c_size_t,                                # workspace workspace_bytes
    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T H HV K V N num_chunks
    c_float, c_int, c_int, c_uint32, c_void_p])
SIGNATURES['gdn_causal_conv1d_bwd'] = (c_int, [
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,   # x weight bias initial_state dy dht
    c_void_p, c_void_p, c_void_p, c_void_p,            # dx dw_part db_part dh0
    c_void_p, c_void_p,                                # cu_seqlens tile_table
    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,   # B T D W N num_tiles stride_x_n stride_x_t
    c_int, c_int, c_int, c_int, c_uint32, c_void_p])
SIGNATURES['gdn_norm_gated_bwd'] = (c_int, [
    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,  # dy x g weight bias
    c_void_p, c_void_p, c_void_p,                      # mean rstd dresidual
    c_void_p, c_void_p, c_void_p, c_void_p,            # dx dg dw_part db_part
    c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_void_p])   # T D ld parts ...
SIGNATURES['gdn_calib_rmw'] = (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p])
CHUNK_STATIC_WORKSPACE_BYTES = 64 << 20
CONV_BWD_TILES_PER_PART = 8

_lib = None
_lock = threading.Lock()


class GDNLibraryError(ImportError):
    pass


def load() -> ctypes.CDLL:
    """Load the HIP library.  Fails loudly when it has not been built: there is no
    fallback implementation behind this package."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise GDNLibraryError(
                f'{LIB_PATH} is missing. Build it with '
                f'`python {os.path.join(os.path.dirname(_HERE), "build.py")}` (needs hipcc); '
                'fla_hip has no CPU or eager fallback.')
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)        # AttributeError if the .so is stale
            fn.restype = res
            fn.argtypes = args
        got = lib.gdn_hip_abi_version()
        if got != ABI_VERSION:
            raise GDNLibraryError(f'{LIB_PATH} has ABI version {got}, expected {ABI_VERSION}; rebuild it')
        _lib = lib
    return _lib


def last_error() -> str:
    msg = load().gdn_last_error()
    return msg.decode() if msg else ''


def check(status: int) -> None:
    """Map C status codes to the exception types the reference raises from Python."""
    if status == GDN_OK:
        return
    msg = last_error()
    if status == GDN_ERR_INVALID:
        raise ValueError(msg)
    if status == GDN_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(f'libgdn_hip status {status}: {msg}')
