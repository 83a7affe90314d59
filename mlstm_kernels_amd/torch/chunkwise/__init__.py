from .hip_xl_chunk import mlstm_chunkwise__hip_xl_chunk, mlstm_siging_chunkwise__hip_xl_chunk

registry = {
    "hip_xl_chunk": mlstm_chunkwise__hip_xl_chunk,
    "hip_xl_chunk_siging": mlstm_siging_chunkwise__hip_xl_chunk,
}
