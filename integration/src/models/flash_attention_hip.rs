//! The `HIP` arm of `fused_attention_ex` (`src/models/flash_attention.rs:348-702`) and of
//! `ViT::forward_with` (`src/models/vit.rs:119-121`), as the lines to add.  Shipped as source.
//!
//! In `fused_attention_ex`, next to the CUDA gates (`:405-472`):
//!
//! ```ignore
//! let hip_dev = dev.starts_with("HIP");
//! let hip_ok = hip_dev && crate::runtime::hip_flash::supported(b, h, n, d);
//! let hip_sage = quantized && hip_ok && settings.tensor_cores && (dt == dtype::FLOAT32 || dt == dtype::BFLOAT16);
//! let hip_bf16 = !hip_sage && hip_ok && dt == dtype::BFLOAT16 && settings.tensor_cores;
//! let hip_f32 = !hip_sage && hip_ok && dt == dtype::FLOAT32;   // CDNA4 has no TF32 MFMA: f32 runs exact
//! if quantized && hip_dev && !hip_sage { note_sage_unsupported(); }
//! if !sage && !bf16 && !tc && !cuda && !cl && !metal && !hip_sage && !hip_bf16 && !hip_f32 { return None; }
//! ```
//!
//! and where the CUDA arms build their `HostCall` (`:560-694`), `hip_calls` below replaces the
//! single `call`; the tail (`:696-701`) captures and executes every element:
//!
//! ```ignore
//! for mut call in calls {
//!     call.device = crate::runtime::device::canonicalize_device_name(&dev);
//!     sess.capture_host(call.clone());
//!     call.exec();
//! }
//! ```
//!
//! `out` needs no host-side zero fill on this device (the kernels write every element), so
//! `Tensor::empty(..).to_param()` replaces the `from_slice(&vec![0.0; ..])` of `:514-530`.
//!
//! In `ViT::forward_with` (`vit.rs:119-121`): `|| d.starts_with("HIP")`.
//!
//! In `fused_attention_train` / `fused_attention_backward` (`:789-977`): accept `dev.starts_with("HIP")`
//! beside `"CUDA"`, `supports(n, d)` becomes `d == 64 || d == 128`, and the launches become
//! `hip_flash::host_call_train_fwd` / `hip_flash::host_calls_train_bwd` (same buffers, same order;
//! `dk`/`dv` need no zero fill: the GQA sum happens inside the kernel).

use crate::engine::session::HostCall;
use crate::runtime::buffer::Buffer;
use crate::runtime::hip_flash::{self, Options, SageOptions, SageScratch};

/// Which HIP kernel family the gates chose.
pub enum HipKernel {
    F32,
    Bf16,
    Sage { bf16_in: bool, scratch: SageScratch, opts: SageOptions },
}

/// The launches of one fused attention call on a HIP device.  `bufs` is
/// `[q, k, v, out, mask-or-out]` exactly as for the CUDA arms (`flash_attention.rs:531-540`).
/// `lens` is the realised int32 `[b]` buffer of per-batch key lengths, if the caller has a
/// key-padding mask in that form (the CUDA arms send such masks to the general path,
/// `flash_attention.rs:389-396`); it selects the `_lens` entry points.
#[allow(clippy::too_many_arguments)]
pub fn hip_calls(dev: &str, kernel: HipKernel, bufs: Vec<Buffer>, lens: Option<Buffer>, b: i64, h: i64, n: i64, d: i64,
                 opts: Options) -> Vec<HostCall> {
    match kernel {
        HipKernel::F32 => {
            hip_flash::note_selected(0);
            vec![hip_flash::host_call_f32(dev, bufs, lens, b, h, n, d, opts)]
        }
        HipKernel::Bf16 => {
            hip_flash::note_selected(1);
            vec![hip_flash::host_call_bf16(dev, bufs, lens, b, h, n, d, opts)]
        }
        HipKernel::Sage { bf16_in, scratch, opts: sage } => {
            hip_flash::note_selected(2);
            let [q, k, v, o, m]: [Buffer; 5] = bufs.try_into().unwrap_or_else(|_| panic!("TGERR: sage expects 5 buffers"));
            hip_flash::host_calls_sage(dev, q, k, v, o, m, lens, scratch, bf16_in, b, h, n, d, opts, sage)
        }
    }
}
