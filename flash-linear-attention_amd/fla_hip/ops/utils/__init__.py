from fla_hip.ops.utils.constant import RCP_LN2
from fla_hip.ops.utils.index import prepare_chunk_indices, prepare_chunk_offsets, prepare_lens, prepare_scan_tables

__all__ = ['RCP_LN2', 'prepare_chunk_indices', 'prepare_chunk_offsets', 'prepare_lens', 'prepare_scan_tables']
