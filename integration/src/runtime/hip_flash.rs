//! Fused attention on the `HIP` device: the `host_call` builders that stand where
//! `cuda_flash::host_call`, `cuda_flash_bf16::host_call` and `cuda_flash_sage::host_call` stand
//! for CUDA (`src/runtime/cuda_flash.rs:283-304`, `cuda_flash_bf16.rs:580-599`,
//! `cuda_flash_sage.rs:487-535`).  Shipped as source; see `ops_hip.rs` for how it was checked.
//!
//! The kernels live in a prebuilt gfx950 code object (`attn_kernels.hsaco`, built from
//! `csrc/attn_entry.hip`).  A `HostCall`'s `src` is that file's path, its `name` one of the entry
//! points below, and `exec` launches it through `Compiled::run_host_kernel` unchanged.
//!
//! | entry                | block | grid                    | arguments after the buffers                  |
//! |----------------------|-------|-------------------------|----------------------------------------------|
//! | `ar_flash_f32`       | 256   | `[ceil(n/128), b*h, 1]` | `n, head_dim, causal, has_mask, hq, hkv`     |
//! | `ar_flash_f32_short` | 256   | `[ceil(n/32), b*h, 1]`  | same; few, short heads; `head_dim` 64        |
//! | `ar_flash_bf16`      | 256   | `[ceil(n/128), b*h, 1]` | same                                         |
//! | `ar_flash_bf16_long` | 512   | `[ceil(n/256), b*h, 1]` | same (`has_mask` must be 0)                  |
//! | `ar_flash_bf16_mid`  | 256   | `[ceil(n/128), b*h, 1]` | same; the pipelined kernel with 4 waves      |
//! | `ar_flash_sage`      | 256   | `[ceil(n/128), b*h, 1]` | same `+ bq, bk`; buffers `+ SQ, SK`; O is f32|
//! | `ar_flash_sage_long` | 512   | `[ceil(n/256), b*h, 1]` | same `+ bq, bk, out_f32`                     |
//! | `ar_flash_sage_mid`  | 256   | `[ceil(n/128), b*h, 1]` | same; the pipelined kernel with 4 waves      |
//! | `ar_flash_sage_qf_long`, `ar_flash_sage_qf_mid`, `ar_flash_sage_fp8_qf_long`, `ar_flash_sage_fp8_qf_mid` | as `_long` / `_mid` | first buffer: the bf16 queries themselves; `SQ` is written (`bq` 128, `bk` 64·2^j) |
//! | `ar_flash_sage_qr_long`, `ar_flash_sage_qr_mid` | as `_long` / `_mid` | first buffer: the f32 queries themselves; `SQ` `[b*h, n]` is written (`bq` 1, `bk` a power of two below 64) |
//! | `ar_flash_sage_fp8`, `ar_flash_sage_fp8_long`, `ar_flash_sage_fp8_mid` | as the int8 entries, on E4M3 codes (`SageOptions::fp8`) |
//! | `<entry>_lens`       | as `<entry>` | as `<entry>`     | one more buffer after the mask slot: `L`, int32 `[b]` key lengths |
//!
//! Key-padding masks: the CUDA fused kernels admit a dense `[n, n]` mask only
//! (`src/models/flash_attention.rs:389-396`); here a per-batch key length keeps a padded batch on the
//! fused kernels.  Every builder takes `lens: Option<Buffer>`; with `Some`, the `_lens` twin of the
//! entry is named and the buffer is inserted after the mask slot.  `ar_flash_f32_short` has no twin: the
//! builder falls through to `ar_flash_f32_lens` then.
//!
//! Unlike the CUDA Sage kernel, which quantises inside the attention kernel (K once per query
//! block, `cuda_flash_sage.rs:248-278`), the K quantiser is a pre-pass of its own here, with K
//! smoothing and per-block scales (128 query tokens / 64 key tokens by default); the queries are
//! quantised by the attention kernel itself where an entry for it exists (`_qf_`: bf16 tensors with
//! `block_q` 128; `_qr_`: f32 tensors with a scale per query, the CUDA kernel's convention, whose K
//! quantiser and V cast are the one launch `ar_sage_quant_rows_cast_f32`).  A Sage call is
//! therefore a short sequence of `HostCall`s; their scratch buffers ride in `bufs`, so a JIT
//! replay finds them again.

use crate::dtype::{self, DTypeId};
use crate::engine::session::HostCall;
use crate::runtime::buffer::Buffer;
use std::sync::atomic::{AtomicU64, Ordering};

/// Path of the code object: `$AUTORUST_HIP_KERNELS`, else next to the executable.
pub fn src() -> String {
    if let Some(p) = crate::helpers::env::get_os("AUTORUST_HIP_KERNELS") {
        return p.to_string_lossy().into_owned();
    }
    let exe = std::env::current_exe().ok();
    let dir = exe.as_deref().and_then(|p| p.parent()).unwrap_or(std::path::Path::new("."));
    dir.join("attn_kernels.hsaco").to_string_lossy().into_owned()
}

/// Per-call switches, as `cuda_flash_bf16::Options` (`cuda_flash_bf16.rs:463-476`).
#[derive(Clone, Copy, Debug)]
pub struct Options {
    pub causal: bool,
    pub has_mask: bool,
    pub h_kv: i64,
}

/// Sage quantiser settings (extensions of this device; block 1 / no smoothing reproduces the
/// CUDA kernel's per-row rule, `cuda_flash_sage.rs:209-222`).
#[derive(Clone, Copy, Debug)]
pub struct SageOptions {
    pub block_q: i64,
    pub block_k: i64,
    pub smooth_k: bool,
    /// E4M3 codes instead of int8 (the CUDA source's `fp8` flag, `cuda_flash_sage.rs:82-84`).
    pub fp8: bool,
}

impl Default for SageOptions {
    fn default() -> Self {
        SageOptions { block_q: 128, block_k: 64, smooth_k: true, fp8: false }
    }
}

/// `supports` / `supported` gates (`cuda_flash.rs:145-147`, `cuda_flash_bf16.rs:431-441`,
/// `cuda_flash_sage.rs:69-74`): head_dim 64 or 128, any n > 0, and a grid that fits.
pub fn supported(b: i64, h: i64, n: i64, d: i64) -> bool {
    n > 0 && n <= 1 << 24 && (d == 64 || d == 128) && b > 0 && h > 0 && b * h <= 65535
}

static SELECTED: [AtomicU64; 3] = [AtomicU64::new(0), AtomicU64::new(0), AtomicU64::new(0)];

/// Which kernel family a call went to: 0 fp32 exact, 1 bf16, 2 Sage int8.
pub fn note_selected(kind: usize) {
    SELECTED[kind].fetch_add(1, Ordering::Relaxed);
    static ONCE: [std::sync::Once; 3] = [std::sync::Once::new(), std::sync::Once::new(), std::sync::Once::new()];
    ONCE[kind].call_once(|| {
        if crate::helpers::env::get_os("AUTORUST_ATTN_DEBUG").is_some() {
            eprintln!(
                "{}",
                [
                    "[attention] flash: fp32 exact, fp32 MFMA (gfx950)",
                    "[attention] flash: bf16 MFMA, software-pipelined for long sequences (gfx950)",
                    "[attention] sage: int8 MFMA for q.k^T, bf16 MFMA for p.v, K smoothing + block scales (gfx950)",
                ][kind]
            );
        }
    });
}

/// Calls dispatched to a kernel family since process start (`cuda_flash_bf16.rs:458-461`).
pub fn selections(kind: usize) -> u64 {
    SELECTED[kind].load(Ordering::Relaxed)
}

fn signature(buf_types: &[DTypeId], nvals: usize, wide: &[usize]) -> Vec<(i64, DTypeId)> {
    let mut s: Vec<(i64, DTypeId)> = buf_types.iter().enumerate().map(|(i, t)| (i as i64, *t)).collect();
    for i in 0..nvals {
        let t = if wide.contains(&i) { dtype::INT64 } else { dtype::INT32 };
        s.push(((buf_types.len() + i) as i64, t));
    }
    s
}

#[allow(clippy::too_many_arguments)]
fn call(name: &str, bufs: Vec<Buffer>, buf_types: &[DTypeId], global: [i64; 3], local: [i64; 3], vals: Vec<i64>, wide: &[usize]) -> HostCall {
    HostCall {
        device: "HIP".into(),
        src: src(),
        name: name.to_string(),
        signature: signature(buf_types, vals.len(), wide),
        bufs,
        global,
        local: Some(local),
        vals,
    }
}

/// The attention launch itself: with key lengths, the `_lens` twin with `L` (int32 `[b]`) after the
/// mask slot (index 4 in every forward entry).
#[allow(clippy::too_many_arguments)]
fn attn_call(name: &str, mut bufs: Vec<Buffer>, buf_types: &[DTypeId], lens: Option<Buffer>, global: [i64; 3], local: [i64; 3],
             vals: Vec<i64>) -> HostCall {
    match lens {
        None => call(name, bufs, buf_types, global, local, vals, &[]),
        Some(l) => {
            let mut types = buf_types.to_vec();
            bufs.insert(5, l);
            types.insert(5, dtype::INT32);
            call(&format!("{name}_lens"), bufs, &types, global, local, vals, &[])
        }
    }
}

fn vals(n: i64, d: i64, h: i64, opts: Options) -> Vec<i64> {
    // `cuda_flash_bf16.rs:550-561`, with the head size as a real parameter
    vec![n, d, opts.causal as i64, opts.has_mask as i64, h, opts.h_kv]
}

/// The software-pipelined kernels serve every launch without an additive mask whose K/V they can address
/// with 32-bit byte offsets ...
fn long_variant(n: i64, d: i64) -> bool {
    (n + 320) * d * 2 < 1 << 31
}

/// ... and run with 4 waves / 128 queries per workgroup (`_mid`: two workgroups per compute unit, one's
/// prologue and epilogue under the other's tiles) where a workgroup sees few tiles, and always at
/// `head_dim` 64.
fn mid_variant(dev: &str, b: i64, h: i64, n: i64, d: i64, causal: bool, has_lens: bool) -> bool {
    if d == 64 || b * h * ((n + 255) / 256) < 2 * crate::runtime::ops_hip::compute_units(dev) {
        return true;
    }
    n <= 1024 || (n <= 2048 && causal && !has_lens)
}

/// The fp32 kernels take 128 queries (keys) per workgroup when that still fills the chip, else 32
/// with the tiles of the other side dealt out between the waves (`*_short`, `head_dim` 64).
fn short_f32(dev: &str, b: i64, heads: i64, n: i64, d: i64) -> bool {
    d == 64 && b * heads * ((n + 127) / 128) < 2 * crate::runtime::ops_hip::compute_units(dev)
}

/// fp32 exact mode: `bufs = [q, k, v, o, mask-or-o]`, all f32 `[b, h, n, d]`; `lens`: int32 `[b]` key lengths.
#[allow(clippy::too_many_arguments)]
pub fn host_call_f32(dev: &str, bufs: Vec<Buffer>, lens: Option<Buffer>, b: i64, h: i64, n: i64, d: i64, opts: Options) -> HostCall {
    let f = dtype::FLOAT32;
    if lens.is_none() && short_f32(dev, b, h, n, d) {
        call("ar_flash_f32_short", bufs, &[f, f, f, f, f], [(n + 31) / 32, b * h, 1], [256, 1, 1], vals(n, d, h, opts), &[])
    } else {
        attn_call("ar_flash_f32", bufs, &[f, f, f, f, f], lens, [(n + 127) / 128, b * h, 1], [256, 1, 1], vals(n, d, h, opts))
    }
}

/// bf16: `bufs = [q, k, v, o, mask-or-o]`, q/k/v/o bf16, mask f32 `[n, n]`; `lens`: int32 `[b]` key lengths.
#[allow(clippy::too_many_arguments)]
pub fn host_call_bf16(dev: &str, bufs: Vec<Buffer>, lens: Option<Buffer>, b: i64, h: i64, n: i64, d: i64, opts: Options) -> HostCall {
    let (bf, f) = (dtype::BFLOAT16, dtype::FLOAT32);
    if !opts.has_mask && long_variant(n, d) && mid_variant(dev, b, h, n, d, opts.causal, lens.is_some()) {
        attn_call("ar_flash_bf16_mid", bufs, &[bf, bf, bf, bf, f], lens, [(n + 127) / 128, b * h, 1], [256, 1, 1], vals(n, d, h, opts))
    } else if !opts.has_mask && long_variant(n, d) {
        attn_call("ar_flash_bf16_long", bufs, &[bf, bf, bf, bf, f], lens, [(n + 255) / 256, b * h, 1], [512, 1, 1], vals(n, d, h, opts))
    } else {
        attn_call("ar_flash_bf16", bufs, &[bf, bf, bf, bf, f], lens, [(n + 127) / 128, b * h, 1], [256, 1, 1], vals(n, d, h, opts))
    }
}

/// Scratch tensors of one Sage call; the dispatcher allocates them (uninitialised is enough)
/// and passes their realised buffers.
pub struct SageScratch {
    pub q8: Buffer,   // int8 [b, h, n, d]
    pub k8: Buffer,   // int8 [b, hkv, n, d]
    pub sq: Buffer,   // f32 [b, h, ceil(n / block_q)]
    pub sk: Buffer,   // f32 [b, hkv, ceil(n / block_k)]
    pub mean: Buffer, // f32 [b, hkv, d]
    pub part: Buffer, // f32 [b, hkv, ceil(n / 64), d]  (partial sums of the K mean)
    pub vb: Option<Buffer>,  // bf16 copy of v when the tensors are f32
    pub o32: Option<Buffer>, // f32 result when the tensors are bf16 and the general kernel runs
}

/// One quantiser launch: per-row scales (`blk == 1`) or per-block scales.  A free function (it returns
/// the launch instead of pushing it) so that the caller's vector is never borrowed across calls.
#[allow(clippy::too_many_arguments)]
fn quant_call(fmt: &str, sfx: &str, x: DTypeId, src: &Buffer, dst: &Buffer, scales: &Buffer, mean: &Buffer, b: i64, heads: i64,
              n: i64, d: i64, blk: i64, nblk: i64, smooth: bool) -> HostCall {
    let (f, i8t) = (dtype::FLOAT32, dtype::INT8);
    let bufs = vec![src.clone(), dst.clone(), scales.clone(), mean.clone()];
    if blk == 1 {
        let rows = b * heads * n;
        let rpb = 256 / (d / 8);
        call(&format!("ar_sage_quant_rows_{fmt}{sfx}"), bufs, &[x, i8t, f, f], [(rows + rpb - 1) / rpb, 1, 1], [256, 1, 1],
             vec![n, d, rows, smooth as i64], &[2])
    } else {
        call(&format!("ar_sage_quant_blocks_{fmt}{sfx}"), bufs, &[x, i8t, f, f], [nblk, b * heads, 1], [256, 1, 1],
             vec![n, d, blk, nblk, smooth as i64], &[])
    }
}

/// Sage int8: the launches of one call, in order.  `q, k, v, o` are f32 or bf16 (`bf16_in`),
/// `mask` is the f32 `[n, n]` additive mask or `o` again; `lens`: int32 `[b]` key lengths.
#[allow(clippy::too_many_arguments)]
pub fn host_calls_sage(
    dev: &str,
    q: Buffer,
    k: Buffer,
    v: Buffer,
    o: Buffer,
    mask: Buffer,
    lens: Option<Buffer>,
    s: SageScratch,
    bf16_in: bool,
    b: i64,
    h: i64,
    n: i64,
    d: i64,
    opts: Options,
    sage: SageOptions,
) -> Vec<HostCall> {
    let (f, bf, i8t) = (dtype::FLOAT32, dtype::BFLOAT16, dtype::INT8);
    let x = if bf16_in { bf } else { f };
    let sfx = if bf16_in { "bf16" } else { "f32" };
    let q8fmt = if sage.fp8 { "fp8_" } else { "" };
    let (general, long) = if sage.fp8 { ("ar_flash_sage_fp8", "ar_flash_sage_fp8_long") } else { ("ar_flash_sage", "ar_flash_sage_long") };
    let hk = opts.h_kv;
    let (bq, bk) = (sage.block_q, sage.block_k);
    let (nqb, nkb, nchunk) = ((n + bq - 1) / bq, (n + bk - 1) / bk, (n + 63) / 64);
    let mut calls = Vec::new();
    let tile_uniform = bk >= 64 && bk % 64 == 0 && (bk / 64).count_ones() == 1;
    // scales over a power of two of keys below 64 (the CUDA kernel's bk = 1) are applied per logit
    let key_scales = bk >= 1 && bk < 64 && bk.count_ones() == 1;
    let pipelined = !opts.has_mask && (tile_uniform || key_scales) && long_variant(n, d);
    // bf16 queries with scales over blocks of 128 are quantised by the attention kernel itself (as the CUDA
    // kernel does): one launch and one pass over Q fewer
    let q_fused = pipelined && tile_uniform && bf16_in && bq == 128;
    // f32 queries with a scale each and K scales per key (the CUDA kernel's own convention): the same, row by row
    let q_rows = pipelined && key_scales && !bf16_in && bq == 1 && !sage.fp8;
    if !q_fused && !q_rows {
        calls.push(quant_call(q8fmt, sfx, x, &q, &s.q8, &s.sq, &s.mean, b, h, n, d, bq, nqb, false));
    }
    if sage.smooth_k {
        let cpb = 256 / (d / 8);
        calls.push(call(&format!("ar_sage_kmean_partial_{sfx}"), vec![k.clone(), s.part.clone()], &[x, f],
                        [(nchunk + cpb - 1) / cpb, b * hk, 1], [256, 1, 1], vec![n, d, nchunk], &[]));
        calls.push(call("ar_sage_kmean_final", vec![s.part.clone(), s.mean.clone()], &[f, f], [b * hk, 1, 1], [d, 1, 1],
                        vec![n, d, nchunk], &[]));
    }
    // unsmoothed f32 K with a scale per key and the cast of V are one launch (ar_sage_quant_rows_cast_f32)
    let kv_one_launch = !bf16_in && bk == 1 && !sage.smooth_k && !sage.fp8 && s.vb.is_some();
    if !kv_one_launch {
        calls.push(quant_call(q8fmt, sfx, x, &k, &s.k8, &s.sk, &s.mean, b, hk, n, d, bk, nkb, sage.smooth_k));
    }
    let vb = match &s.vb {
        Some(vb) if kv_one_launch => {
            let rows = b * hk * n;
            let rpb = 256 / (d / 8);
            let (row_blocks, nv) = ((rows + rpb - 1) / rpb, rows * d);
            calls.push(call("ar_sage_quant_rows_cast_f32", vec![k.clone(), s.k8.clone(), s.sk.clone(), v.clone(), vb.clone()],
                            &[f, i8t, f, f, bf], [row_blocks + ((nv + 255) / 256).min(16384), 1, 1], [256, 1, 1],
                            vec![n, d, rows, nv, row_blocks], &[2, 3]));
            vb.clone()
        }
        Some(vb) => {
            let nv = b * hk * n * d;
            calls.push(call("ar_cast_bf16", vec![v.clone(), vb.clone()], &[f, bf], [((nv + 255) / 256).min(16384), 1, 1], [256, 1, 1],
                            vec![nv], &[0]));
            vb.clone()
        }
        None => v.clone(),
    };
    let mut sv = vals(n, d, h, opts);
    sv.push(bq);
    sv.push(bk);
    if pipelined {
        sv.push(!bf16_in as i64); // out_f32
        let mid = mid_variant(dev, b, h, n, d, opts.causal, lens.is_some());
        let (grid, block) = if mid { ([(n + 127) / 128, b * h, 1], [256, 1, 1]) } else { ([(n + 255) / 256, b * h, 1], [512, 1, 1]) };
        if q_fused {
            // Q itself in the first slot; the scales slot is written
            let name = match (sage.fp8, mid) {
                (false, true) => "ar_flash_sage_qf_mid",
                (false, false) => "ar_flash_sage_qf_long",
                (true, true) => "ar_flash_sage_fp8_qf_mid",
                (true, false) => "ar_flash_sage_fp8_qf_long",
            };
            calls.push(attn_call(name, vec![q, s.k8, vb, o, mask, s.sq, s.sk], &[bf, i8t, bf, x, f, f, f], lens, grid, block, sv));
        } else if q_rows {
            let name = if mid { "ar_flash_sage_qr_mid" } else { "ar_flash_sage_qr_long" };
            calls.push(attn_call(name, vec![q, s.k8, vb, o, mask, s.sq, s.sk], &[f, i8t, bf, x, f, f, f], lens, grid, block, sv));
        } else {
            let name = if mid { if sage.fp8 { "ar_flash_sage_fp8_mid" } else { "ar_flash_sage_mid" } } else { long };
            calls.push(attn_call(name, vec![s.q8, s.k8, vb, o, mask, s.sq, s.sk], &[i8t, i8t, bf, x, f, f, f], lens, grid, block, sv));
        }
    } else if !bf16_in {
        calls.push(attn_call(general, vec![s.q8, s.k8, vb, o, mask, s.sq, s.sk], &[i8t, i8t, bf, f, f, f, f], lens,
                             [(n + 127) / 128, b * h, 1], [256, 1, 1], sv));
    } else {
        // the general kernel stores f32 (the CUDA kernel's convention); bf16 tensors get their
        // bf16 result through one more cast
        let o32 = s.o32.expect("o32 scratch for bf16 tensors");
        let m2 = if opts.has_mask { mask } else { o32.clone() };
        calls.push(attn_call(general, vec![s.q8, s.k8, vb, o32.clone(), m2, s.sq, s.sk], &[i8t, i8t, bf, f, f, f, f], lens,
                             [(n + 127) / 128, b * h, 1], [256, 1, 1], sv));
        let no = b * h * n * d;
        calls.push(call("ar_cast_bf16", vec![o32, o], &[f, bf], [((no + 255) / 256).min(16384), 1, 1], [256, 1, 1], vec![no], &[0]));
    }
    calls
}

// ---- training (counterpart of `cuda_flash_train::{run_fwd, run_prep, run_dq, run_dkv}`,
// src/runtime/cuda_flash_train.rs:336-541): f32 tensors, dense `[b, h, n, d]` ----

/// Forward that also writes `lse [b*h, n]`: `bufs = [q, k, v, o, lse, mask-or-o]`.
pub fn host_call_train_fwd(dev: &str, bufs: Vec<Buffer>, b: i64, h: i64, n: i64, d: i64, opts: Options) -> HostCall {
    let f = dtype::FLOAT32;
    if short_f32(dev, b, h, n, d) {
        call("ar_fl_fwd_short", bufs, &[f, f, f, f, f, f], [(n + 31) / 32, b * h, 1], [256, 1, 1], vals(n, d, h, opts), &[])
    } else {
        call("ar_fl_fwd", bufs, &[f, f, f, f, f, f], [(n + 127) / 128, b * h, 1], [256, 1, 1], vals(n, d, h, opts), &[])
    }
}

/// The three launches of the backward, in order.  `delta` is a scratch tensor `[b*h, n]`; `mask` is
/// the additive mask or `dq` again (the reference's dummy, cuda_flash_train.rs:442-449).
#[allow(clippy::too_many_arguments)]
pub fn host_calls_train_bwd(
    dev: &str,
    q: Buffer, k: Buffer, v: Buffer, o: Buffer, lse: Buffer, dout: Buffer, mask: Buffer, delta: Buffer,
    dq: Buffer, dk: Buffer, dv: Buffer, b: i64, h: i64, n: i64, d: i64, opts: Options,
) -> Vec<HostCall> {
    let f = dtype::FLOAT32;
    let short = short_f32(dev, b, opts.h_kv, n, d);
    let tiles = if short { (n + 31) / 32 } else { (n + 127) / 128 };
    let (dq_name, dkv_name) = if short { ("ar_fl_bwd_dq_short", "ar_fl_bwd_dkv_short") } else { ("ar_fl_bwd_dq", "ar_fl_bwd_dkv") };
    vec![
        call("ar_fl_prep", vec![o, dout.clone(), delta.clone()], &[f, f, f], [(n + 3) / 4, b * h, 1], [256, 1, 1], vec![n, d], &[]),
        call(dq_name, vec![q.clone(), k.clone(), v.clone(), dout.clone(), lse.clone(), delta.clone(), mask.clone(), dq],
             &[f, f, f, f, f, f, f, f], [tiles, b * h, 1], [256, 1, 1], vals(n, d, h, opts), &[]),
        call(dkv_name, vec![q, k, v, dout, lse, delta, mask, dk, dv],
             &[f, f, f, f, f, f, f, f, f], [tiles, b * opts.h_kv, 1], [256, 1, 1], vals(n, d, h, opts), &[]),
    ]
}
