//! W4A16 GEMM for AMD Instinct MI355X behind kiln's `kiln-marlin-gemm` interface.
//!
//! Same public surface as the crate it replaces (`marlin_w4a16_gemm`, `pack::MAX_Q`,
//! `pack::Q_OFFSET`, `pack::quantize_and_pack`), so `kiln-model/src/marlin_proj.rs` builds
//! unchanged.  Differences that stay inside this crate:
//!   * activations and output are bf16 end to end (no fp16 round trip);
//!   * `b_packed` / `scales` carry the tile layout of the HIP kernels (same shapes,
//!     `[k/16, 2n]` i32 and `[k/g, n]` f16; contents are opaque to callers);
//!   * the workspace is sized by `kiln_w4a16_workspace_bytes`, kept per (device, stream) and
//!     grown on demand; only its counter prefix (`kiln_w4a16_workspace_zeroed_bytes`) is ever
//!     cleared, once, when the buffer is allocated -- no memset rides in front of a GEMM.
//! All arithmetic lives behind the C ABI declared in `include/kiln_w4a16.h`.
//!
//! Written without a Rust toolchain at hand: the storage accessors follow candle 0.10's
//! CUDA-style API (`as_cuda_slice`, `device_ptr`) and must be pointed at whatever
//! HIP-capable storage the host build of candle exposes.

use candle_core::{backend::BackendStorage, cuda_backend::cudarc::driver::DevicePtr, DType, Result, Tensor};
use core::ffi::c_void;
use half::{bf16, f16};
use std::collections::HashMap;
use std::sync::{Mutex, OnceLock};

unsafe extern "C" {
    fn kiln_marlin_w4a16_gemm(
        a: *const c_void, b: *const c_void, c: *mut c_void, s: *const c_void,
        prob_m: i32, prob_n: i32, prob_k: i32, workspace: *mut c_void, groupsize: i32,
        dev: i32, stream: *mut c_void, thread_k: i32, thread_n: i32, sms: i32, max_par: i32,
    ) -> i32;
    fn kiln_w4a16_workspace_bytes(prob_m: i32, prob_n: i32, prob_k: i32) -> usize;
    fn kiln_w4a16_workspace_zeroed_bytes() -> usize;
    fn kiln_w4a16_quantize_and_pack(
        weight: *const f32, k: i32, n: i32, groupsize: i32,
        b_packed: *mut i32, scales_f16: *mut u16, dequant: *mut f32,
    ) -> i32;
    fn kiln_w4a16_quantize_and_pack_device(
        weight_bf16: *const c_void, k: i32, n: i32, groupsize: i32,
        b_packed: *mut c_void, scales_f16: *mut c_void, dev: i32, stream: *mut c_void,
    ) -> i32;
}

macro_rules! device_slice {
    ($tensor:expr, $ty:ty, $what:literal) => {{
        let (storage, layout) = $tensor.storage_and_layout();
        match &*storage {
            candle_core::Storage::Cuda(c) => (c.as_cuda_slice::<$ty>()?.slice(layout.start_offset()..), c.device().clone()),
            _ => candle_core::bail!(concat!("kiln-marlin-gemm: ", $what, " must be on the GPU")),
        }
    }};
}

/// `[m, k] bf16 x dequant([k/16, 2n] i32, [k/g, n] f16) -> [m, n] bf16`; `groupsize` is -1 or 128.
pub fn marlin_w4a16_gemm(a: &Tensor, b_packed: &Tensor, scales: &Tensor, groupsize: i32) -> Result<Tensor> {
    let (m, k) = a.dims2()?;
    let (b_rows, b_cols) = b_packed.dims2()?;
    let (s_rows, n) = scales.dims2()?;
    if k % 128 != 0 { candle_core::bail!("kiln-marlin-gemm: k must be a multiple of 128 (got {k})"); }
    if n % 256 != 0 { candle_core::bail!("kiln-marlin-gemm: n must be a multiple of 256 (got {n})"); }
    if (b_rows, b_cols) != (k / 16, n * 2) {
        candle_core::bail!("kiln-marlin-gemm: b_packed shape [{b_rows}, {b_cols}] does not match expected [k/16={}, n*16/8={}] for k={k}, n={n}", k / 16, n * 2);
    }
    if groupsize != -1 && groupsize != 128 { candle_core::bail!("kiln-marlin-gemm: groupsize must be -1 or 128 (got {groupsize})"); }
    let groups = if groupsize == -1 { 1 } else { k / 128 };
    if s_rows != groups { candle_core::bail!("kiln-marlin-gemm: scales rows {s_rows} != expected {groups} (k={k}, groupsize={groupsize})"); }
    if a.dtype() != DType::BF16 { candle_core::bail!("kiln-marlin-gemm: a must be bf16 (got {:?})", a.dtype()); }
    if b_packed.dtype() != DType::I32 { candle_core::bail!("kiln-marlin-gemm: b_packed must be i32 (got {:?})", b_packed.dtype()); }
    if scales.dtype() != DType::F16 { candle_core::bail!("kiln-marlin-gemm: scales must be f16 (got {:?})", scales.dtype()); }

    let (a, b_packed, scales) = (a.contiguous()?, b_packed.contiguous()?, scales.contiguous()?);
    // the kernels write every element of the output: no zero fill
    let out = unsafe { Tensor::empty((m, n), DType::BF16, a.device())? };
    let workspace = workspace_for(&a, m, n, k)?;
    {
        let (a_s, dev) = device_slice!(a, bf16, "a");
        let (b_s, _) = device_slice!(b_packed, i32, "b_packed");
        let (s_s, _) = device_slice!(scales, f16, "scales");
        let (c_s, _) = device_slice!(out, bf16, "c");
        let (w_s, _) = device_slice!(workspace, u8, "workspace");
        let stream = dev.cuda_stream();
        let status = unsafe {
            let (ap, _g0) = a_s.device_ptr(&stream);
            let (bp, _g1) = b_s.device_ptr(&stream);
            let (sp, _g2) = s_s.device_ptr(&stream);
            let (cp, _g3) = c_s.device_ptr(&stream);
            let (wp, _g4) = w_s.device_ptr(&stream);
            kiln_marlin_w4a16_gemm(ap as *const _, bp as *const _, cp as *mut _, sp as *const _,
                m as i32, n as i32, k as i32, wp as *mut _, groupsize, dev.ordinal() as i32,
                stream.cu_stream() as *mut c_void, -1, -1, -1, 16)
        };
        if status != 0 {
            candle_core::bail!("kiln_marlin_w4a16_gemm failed with status {status} (1=ERR_PROB_SHAPE, 2=ERR_KERN_SHAPE, 3=launch, 4=argument) for m={m}, n={n}, k={k}, groupsize={groupsize}");
        }
    }
    Ok(out)
}

/// One workspace per (device ordinal, stream handle).  `kiln_w4a16_workspace_bytes` never
/// decreases with m, so a buffer that served a larger call serves every smaller one; only the
/// counter prefix has to be zero, once: every call leaves it zero again.  Calls that share a
/// workspace are ordered on its stream.
fn workspace_for(a: &Tensor, m: usize, n: usize, k: usize) -> Result<Tensor> {
    static CACHE: OnceLock<Mutex<HashMap<(usize, usize), Tensor>>> = OnceLock::new();
    let need = unsafe { kiln_w4a16_workspace_bytes(m as i32, n as i32, k as i32) };
    let key = {
        let (_, dev) = device_slice!(a, bf16, "a");
        (dev.ordinal(), dev.cuda_stream().cu_stream() as usize)
    };
    let mut cache = CACHE.get_or_init(|| Mutex::new(HashMap::new())).lock().unwrap();
    if let Some(ws) = cache.get(&key) {
        if ws.elem_count() >= need { return Ok(ws.clone()); }
    }
    let zeroed = unsafe { kiln_w4a16_workspace_zeroed_bytes() };
    let head = Tensor::zeros((zeroed,), DType::U8, a.device())?;
    let ws = if need > zeroed {
        let tail = unsafe { Tensor::empty((need - zeroed,), DType::U8, a.device())? };
        Tensor::cat(&[&head, &tail], 0)?
    } else { head };
    cache.insert(key, ws.clone());
    Ok(ws)
}

/// Quantise and pack a bf16 `[k, n]` weight where it lies, on the GPU: the bits `pack::quantize_and_pack`
/// gives for the same values, without the download, host pack and upload.  A caller that holds the weight
/// on the device (`kiln-model/src/marlin_proj.rs:86-181` does) calls this instead of the three phases.
/// Returns `(b_packed [k/16, 2n] i32, scales [k/g, n] f16)`.
pub fn quantize_and_pack_device(weight_bf16: &Tensor, groupsize: i32) -> Result<(Tensor, Tensor)> {
    let (k, n) = weight_bf16.dims2()?;
    if k % 128 != 0 || n % 256 != 0 { candle_core::bail!("kiln-marlin-gemm: weight [{k}, {n}] needs k % 128 == 0 and n % 256 == 0"); }
    if groupsize != -1 && groupsize != 128 { candle_core::bail!("kiln-marlin-gemm: groupsize must be -1 or 128 (got {groupsize})"); }
    if weight_bf16.dtype() != DType::BF16 { candle_core::bail!("kiln-marlin-gemm: weight must be bf16 (got {:?})", weight_bf16.dtype()); }
    let w = weight_bf16.contiguous()?;
    let groups = if groupsize == -1 { 1 } else { k / 128 };
    let b_packed = unsafe { Tensor::empty((k / 16, n * 2), DType::I32, w.device())? };
    let scales = unsafe { Tensor::empty((groups, n), DType::F16, w.device())? };
    {
        let (w_s, dev) = device_slice!(w, bf16, "weight");
        let (b_s, _) = device_slice!(b_packed, i32, "b_packed");
        let (s_s, _) = device_slice!(scales, f16, "scales");
        let stream = dev.cuda_stream();
        let status = unsafe {
            let (wp, _g0) = w_s.device_ptr(&stream);
            let (bp, _g1) = b_s.device_ptr(&stream);
            let (sp, _g2) = s_s.device_ptr(&stream);
            kiln_w4a16_quantize_and_pack_device(wp as *const _, k as i32, n as i32, groupsize, bp as *mut _, sp as *mut _,
                dev.ordinal() as i32, stream.cu_stream() as *mut c_void)
        };
        if status != 0 { candle_core::bail!("kiln_w4a16_quantize_and_pack_device failed with status {status} for k={k}, n={n}"); }
    }
    Ok((b_packed, scales))
}

pub mod pack {
    use super::*;

    pub const MAX_Q: i32 = 15;
    pub const Q_OFFSET: i32 = 8;

    /// Quantise `weight` (row-major `[k, n]`) and pack it for the kernels.
    /// Returns `(b_packed [k*n/8], scales [(k/g)*n], dequant [k*n])` like the crate it replaces.
    pub fn quantize_and_pack(weight: &[f32], k: usize, n: usize, groupsize: i64) -> (Vec<i32>, Vec<f16>, Vec<f32>) {
        assert_eq!(weight.len(), k * n);
        assert_eq!(k % 128, 0, "k must be %128 == 0");
        assert_eq!(n % 256, 0, "n must be %256 == 0");
        let groups = if groupsize == -1 { 1 } else { k / groupsize as usize };
        let mut packed = vec![0i32; k * n / 8];
        let mut scales = vec![0u16; groups * n];
        let mut dequant = vec![0f32; k * n];
        let st = unsafe {
            kiln_w4a16_quantize_and_pack(weight.as_ptr(), k as i32, n as i32, groupsize as i32,
                packed.as_mut_ptr(), scales.as_mut_ptr(), dequant.as_mut_ptr())
        };
        assert_eq!(st, 0, "kiln_w4a16_quantize_and_pack failed with status {st}");
        (packed, scales.into_iter().map(f16::from_bits).collect(), dequant)
    }
}
