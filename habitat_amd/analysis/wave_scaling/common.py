"""Wave sizes of one kernel on two devices, on the host
(analyzer/habitat/analysis/wave_scaling/common.py:3-20).  The batched kernel
computes the same four numbers per record on the GPU; this is the scalar face
of it for callers of the reference's function."""


def calculate_wave_info(kernel, origin_device, dest_device, metadata_manager):
    """(origin wave size, destination wave size, origin occupancy, destination
    occupancy).  A wave size is blocks per multiprocessor times multiprocessors;
    the destination's occupancy uses the register table's count for this kernel
    on that architecture when the table has one."""
    table_regs = metadata_manager.kernel_registers_for(kernel, dest_device)
    dest_args = (dest_device,) if table_regs is None else (dest_device, table_regs)
    occupancies = (kernel.thread_block_occupancy(origin_device),
                   kernel.thread_block_occupancy(*dest_args))
    waves = tuple(device.num_sms * occupancy
                  for device, occupancy in zip((origin_device, dest_device), occupancies))
    return waves + occupancies
