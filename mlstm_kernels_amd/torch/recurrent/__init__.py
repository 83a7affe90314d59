from .hip_step import mlstm_recurrent_sequence__hip, mlstm_recurrent_step__hip, mlstm_recurrent_step__hip_fw

registry_step = {
    "hip": mlstm_recurrent_step__hip,
}

registry_sequence = {
    "native_sequence__hip": mlstm_recurrent_sequence__hip,
}
