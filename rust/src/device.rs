// `src/device.rs` after the switch: the Vulkan modules (buffer_heap, command_buffer, context, descriptor_pool, fence,
// heap, staging, timestamp) are gone; the one device module is the binding of libdescent_hip.so.
pub mod hip;
pub(crate) mod common {
    pub(crate) use super::hip::{BufferId, HipDevice, HipSchedule};
}
