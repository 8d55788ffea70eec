//! `strix-backend-mi355` — AMD Instinct MI355X (gfx950) matmul backend.
//!
//! Binds `libstrix_mi355.so` (hand-written HIP kernels behind the C ABI of
//! `include/strix_mi355.h`) to `strix_core::accel::WeightAccel`, the seam
//! `strix-backend-rocm` implements with `RocmWeightAccel`
//! (crates/strix-backend-rocm/src/decode.rs:2490-3900).  Weights stay resident in
//! HBM; `gemv`, `gemv_batch`, `prefill_q8_gemm`, `lm_head_argmax_rows` and the MoE
//! entry points run on the device, every other trait method keeps its default
//! (`None` / `false`), so the models fall back to their own code for those.
//!
//! The `mi355` feature gates everything; the default build is a stub, like the
//! `rocm` feature of `strix-backend-rocm`.
//!
//! Return convention of the library: 1 done, 0 not resident, < 0 error.  The trait
//! has no error channel (its `bool` / `Option` mean "not adopted, use the CPU"), so
//! errors are logged with `tracing::warn!` and reported as a decline: the model's
//! own CPU matmul then runs, as it does today when the ROCm backend declines.

#[cfg(feature = "mi355")]
mod ffi;

use strix_core::device::{DeviceInfo, DeviceKind};

/// Probe the backend for `device-info`.
pub fn device_info() -> DeviceInfo {
    #[cfg(feature = "mi355")]
    {
        match Mi355WeightAccel::with_device(0) {
            Ok(acc) => {
                let mut i = DeviceInfo::new(DeviceKind::Gpu, acc.adapter_name().to_string(), "mi355");
                i.notes.push("libstrix_mi355.so loaded (gfx950 HIP kernels)".into());
                i
            }
            Err(e) => {
                let mut i = DeviceInfo::new(DeviceKind::Gpu, "MI355X (unavailable)", "mi355");
                i.notes.push(e);
                i
            }
        }
    }
    #[cfg(not(feature = "mi355"))]
    {
        let mut i = DeviceInfo::new(DeviceKind::Gpu, "MI355X (disabled)", "mi355");
        i.notes
            .push("build with --features mi355 to link libstrix_mi355.so".into());
        i
    }
}

#[cfg(feature = "mi355")]
pub use accel::Mi355WeightAccel;

#[cfg(feature = "mi355")]
mod accel {
    use super::ffi;
    use std::collections::HashMap;
    use std::ffi::{CStr, CString};
    use std::os::raw::{c_char, c_float, c_int};
    use std::sync::Mutex;
    use strix_core::accel::WeightAccel;

    /// Shape of an adopted expert layer, needed to size the results of the MoE calls.
    #[derive(Clone, Copy)]
    struct MoeShape {
        hidden: usize,
        #[allow(dead_code)]
        eff: usize,
        #[allow(dead_code)]
        ne: usize,
    }

    /// One queued expert group of the `moe_expert_queue[_q8]` / `moe_expert_flush` pair.
    struct QueuedGroup {
        layer: usize,
        expert: usize,
        rows: usize,
        dy_off: usize,
        xs: Vec<f32>,
    }

    pub struct Mi355WeightAccel {
        ctx: *mut ffi::SmxCtx,
        name: String,
        moe: HashMap<usize, MoeShape>,
        /// One context owns one HIP stream and its scratch buffers: calls are serialised
        /// (`RocmWeightAccel` holds its scratch behind a Mutex the same way, decode.rs:559-562).
        lock: Mutex<()>,
        queue: Mutex<Vec<QueuedGroup>>,
    }

    // The context is only touched under `lock`; the library keeps no thread-local state in it.
    unsafe impl Send for Mi355WeightAccel {}
    unsafe impl Sync for Mi355WeightAccel {}

    fn last_error(ctx: *const ffi::SmxCtx) -> String {
        // valid for ctx == null too: the calling thread's last failed smx_create
        let p = unsafe { ffi::smx_last_error(ctx) };
        if p.is_null() {
            return String::from("unknown error");
        }
        unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned()
    }

    impl Mi355WeightAccel {
        /// Open device 0; `None` when there is no usable GPU or the library fails to start
        /// (the signature of `RocmWeightAccel::new`, decode.rs:565).
        pub fn new() -> Option<Self> {
            match Self::with_device(0) {
                Ok(a) => Some(a),
                Err(e) => {
                    tracing::warn!("mi355: {e}");
                    None
                }
            }
        }

        /// Open a given HIP device; the error text is the library's.
        pub fn with_device(device: i32) -> Result<Self, String> {
            let mut ctx: *mut ffi::SmxCtx = std::ptr::null_mut();
            let rc = unsafe { ffi::smx_create(device as c_int, &mut ctx) };
            if rc != 1 || ctx.is_null() {
                return Err(last_error(std::ptr::null()));
            }
            let name = {
                let p = unsafe { ffi::smx_name(ctx) };
                if p.is_null() {
                    String::from("MI355X")
                } else {
                    unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned()
                }
            };
            Ok(Mi355WeightAccel {
                ctx,
                name,
                moe: HashMap::new(),
                lock: Mutex::new(()),
                queue: Mutex::new(Vec::new()),
            })
        }

        pub fn adapter_name(&self) -> &str {
            &self.name
        }

        /// Device bytes held by resident weights.
        pub fn resident_bytes(&self) -> usize {
            unsafe { ffi::smx_resident_bytes(self.ctx) }
        }

        /// Drop one resident weight (the reference never frees; useful for model switches).
        pub fn evict(&mut self, key: &str) -> bool {
            let Some(k) = cstr(key) else { return false };
            let _g = self.lock.lock().unwrap();
            self.done(unsafe { ffi::smx_evict(self.ctx, k.as_ptr()) })
        }

        /// Top-k routing of one token's router logits on the device (softmax over all
        /// experts, k largest, renormalised): the `topk_router` kernel of
        /// crates/strix-backend-rocm/src/kernels.rs, which feeds the queued MoE of the fused
        /// decode token.
        pub fn moe_route(&self, logits: &[f32], k: usize) -> Option<(Vec<i32>, Vec<f32>)> {
            let mut ids = vec![0i32; k];
            let mut w = vec![0f32; k];
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_moe_route(self.ctx, logits.as_ptr(), logits.len(), k, ids.as_mut_ptr(), w.as_mut_ptr())
            };
            self.done(rc).then_some((ids, w))
        }

        /// 1 -> true, 0 -> false (not resident), < 0 -> log the library's message, false.
        fn done(&self, rc: c_int) -> bool {
            if rc < 0 {
                tracing::warn!("mi355: {}", last_error(self.ctx));
            }
            rc == 1
        }

        fn dims(&self, key: &CStr) -> Option<(usize, usize)> {
            let (mut in_dim, mut out_dim) = (0usize, 0usize);
            let rc = unsafe { ffi::smx_weight_dims(self.ctx, key.as_ptr(), &mut in_dim, &mut out_dim) };
            (rc == 1).then_some((in_dim, out_dim))
        }

        #[allow(clippy::too_many_arguments)]
        fn upload_moe(
            &mut self,
            q6: bool,
            layer: usize,
            gate: &[u8],
            up: &[u8],
            down: &[u8],
            hidden: usize,
            eff: usize,
            ne: usize,
        ) -> bool {
            let rc = {
                let _g = self.lock.lock().unwrap();
                let (g, gn, u, un, d, dn) = (
                    gate.as_ptr().cast(),
                    gate.len(),
                    up.as_ptr().cast(),
                    up.len(),
                    down.as_ptr().cast(),
                    down.len(),
                );
                if q6 {
                    unsafe { ffi::smx_upload_moe_q6(self.ctx, layer, g, gn, u, un, d, dn, hidden, eff, ne) }
                } else {
                    unsafe { ffi::smx_upload_moe_q8(self.ctx, layer, g, gn, u, un, d, dn, hidden, eff, ne) }
                }
            };
            let ok = self.done(rc);
            if ok {
                self.moe.insert(layer, MoeShape { hidden, eff, ne });
            }
            ok
        }

        fn queue_group(&self, layer: usize, e: usize, xs: &[f32], m: usize, dy_off: usize) -> bool {
            let Some(shape) = self.moe.get(&layer) else { return false };
            if m == 0 || xs.len() != m * shape.hidden {
                return false;
            }
            self.queue.lock().unwrap().push(QueuedGroup {
                layer,
                expert: e,
                rows: m,
                dy_off,
                xs: xs.to_vec(),
            });
            true
        }
    }

    fn cstr(key: &str) -> Option<CString> {
        CString::new(key).ok() // a key with an interior NUL is simply not adopted
    }

    impl Drop for Mi355WeightAccel {
        fn drop(&mut self) {
            unsafe { ffi::smx_destroy(self.ctx) }
        }
    }

    impl WeightAccel for Mi355WeightAccel {
        fn upload_q4_0(&mut self, key: &str, bytes: &[u8], in_dim: usize, out_dim: usize) -> bool {
            let Some(k) = cstr(key) else { return false };
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_upload_q4_0(self.ctx, k.as_ptr(), bytes.as_ptr().cast(), bytes.len(), in_dim, out_dim)
            };
            self.done(rc)
        }

        fn upload_q6_k(&mut self, key: &str, bytes: &[u8], in_dim: usize, out_dim: usize) -> bool {
            let Some(k) = cstr(key) else { return false };
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_upload_q6_k(self.ctx, k.as_ptr(), bytes.as_ptr().cast(), bytes.len(), in_dim, out_dim)
            };
            self.done(rc)
        }

        fn upload_q8_0(&mut self, key: &str, bytes: &[u8], in_dim: usize, out_dim: usize) -> bool {
            let Some(k) = cstr(key) else { return false };
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_upload_q8_0(self.ctx, k.as_ptr(), bytes.as_ptr().cast(), bytes.len(), in_dim, out_dim)
            };
            self.done(rc)
        }

        fn upload_moe_q8(
            &mut self,
            layer: usize,
            gate: &[u8],
            up: &[u8],
            down: &[u8],
            hidden: usize,
            eff: usize,
            ne: usize,
        ) -> bool {
            self.upload_moe(false, layer, gate, up, down, hidden, eff, ne)
        }

        fn upload_moe_q6(
            &mut self,
            layer: usize,
            gate: &[u8],
            up: &[u8],
            down: &[u8],
            hidden: usize,
            eff: usize,
            ne: usize,
        ) -> bool {
            self.upload_moe(true, layer, gate, up, down, hidden, eff, ne)
        }

        fn moe_ffn(&self, layer: usize, ids: &[i32], wexp: &[f32], x: &[f32], sgate: f32) -> Option<Vec<f32>> {
            let shape = *self.moe.get(&layer)?;
            if ids.len() != wexp.len() {
                return None;
            }
            let mut y = vec![0f32; shape.hidden];
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_moe_ffn(
                    self.ctx,
                    layer,
                    ids.as_ptr(),
                    wexp.as_ptr(),
                    ids.len(),
                    x.as_ptr(),
                    x.len(),
                    sgate as c_float,
                    y.as_mut_ptr(),
                    y.len(),
                )
            };
            self.done(rc).then_some(y)
        }

        fn prefill_q8_gemm(&self, key: &str, xs: &[f32], m: usize) -> Option<Vec<f32>> {
            let k = cstr(key)?;
            let (in_dim, out_dim) = self.dims(&k)?;
            if m == 0 || xs.len() != m * in_dim {
                return None;
            }
            let mut y = vec![0f32; m * out_dim];
            let _g = self.lock.lock().unwrap();
            let rc = unsafe { ffi::smx_gemm(self.ctx, k.as_ptr(), xs.as_ptr(), m, in_dim, y.as_mut_ptr(), y.len()) };
            self.done(rc).then_some(y)
        }

        fn lm_head_argmax_rows(&self, key: &str, xs: &[f32], m: usize) -> Option<Vec<u32>> {
            let k = cstr(key)?;
            let (in_dim, _) = self.dims(&k)?;
            if m == 0 || xs.len() != m * in_dim {
                return None;
            }
            let mut out = vec![0u32; m];
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_lm_head_argmax_rows(self.ctx, k.as_ptr(), xs.as_ptr(), m, in_dim, out.as_mut_ptr())
            };
            self.done(rc).then_some(out)
        }

        fn moe_expert_ffn(&self, layer: usize, e: usize, xs: &[f32], m: usize) -> Option<Vec<f32>> {
            let shape = *self.moe.get(&layer)?;
            if m == 0 || xs.len() != m * shape.hidden {
                return None;
            }
            let mut y = vec![0f32; m * shape.hidden];
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_moe_expert_ffn(self.ctx, layer, e, xs.as_ptr(), m, y.as_mut_ptr(), y.len())
            };
            self.done(rc).then_some(y)
        }

        fn moe_expert_queue(&self, layer: usize, e: usize, xs: &[f32], m: usize, dy_off: usize) -> bool {
            self.queue_group(layer, e, xs, m, dy_off)
        }

        fn moe_expert_queue_q8(&self, layer: usize, e: usize, xs: &[f32], m: usize, dy_off: usize) -> bool {
            self.queue_group(layer, e, xs, m, dy_off)
        }

        /// Runs every queued group in ONE grouped call and returns the first `rows` rows of the
        /// dy pool (group g's rows at its `dy_off`).  Groups of one layer only, as the models
        /// queue them (a layer's experts, then flush).
        fn moe_expert_flush(&self, rows: usize, hidden: usize) -> Option<Vec<f32>> {
            let mut groups = std::mem::take(&mut *self.queue.lock().unwrap());
            if groups.is_empty() {
                return None;
            }
            let layer = groups[0].layer;
            if groups.iter().any(|g| g.layer != layer) {
                tracing::warn!("mi355: moe_expert_flush with groups of several layers; dropped");
                return None;
            }
            let shape = *self.moe.get(&layer)?;
            if shape.hidden != hidden {
                return None;
            }
            groups.sort_by_key(|g| g.dy_off);
            let total: usize = groups.iter().map(|g| g.rows).sum();
            let mut plan: Vec<i32> = Vec::with_capacity(groups.len() * 2);
            let mut xs: Vec<f32> = Vec::with_capacity(total * hidden);
            for g in &groups {
                plan.push(g.expert as i32);
                plan.push(g.rows as i32);
                xs.extend_from_slice(&g.xs);
            }
            let mut dy = vec![0f32; total * hidden];
            let rc = {
                let _g = self.lock.lock().unwrap();
                unsafe {
                    ffi::smx_moe_layer_ffn(
                        self.ctx,
                        layer,
                        plan.as_ptr(),
                        groups.len(),
                        xs.as_ptr(),
                        total,
                        dy.as_mut_ptr(),
                        dy.len(),
                    )
                }
            };
            if !self.done(rc) {
                return None;
            }
            // scatter the groups to their offsets in the pool
            let mut pool = vec![0f32; rows * hidden];
            let mut src = 0usize;
            for g in &groups {
                let n = g.rows * hidden;
                let dst = g.dy_off * hidden;
                if dst + n > pool.len() {
                    return None;
                }
                pool[dst..dst + n].copy_from_slice(&dy[src..src + n]);
                src += n;
            }
            Some(pool)
        }

        fn moe_layer_ffn(&self, layer: usize, plan: &[(i32, i32)], xs: &[f32], rows: usize) -> Option<Vec<f32>> {
            let shape = *self.moe.get(&layer)?;
            if rows == 0 || xs.len() != rows * shape.hidden {
                return None;
            }
            let flat: Vec<i32> = plan.iter().flat_map(|&(e, n)| [e, n]).collect(); // (expert, rows of the group)
            let mut dy = vec![0f32; rows * shape.hidden];
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_moe_layer_ffn(
                    self.ctx,
                    layer,
                    flat.as_ptr(),
                    plan.len(),
                    xs.as_ptr(),
                    rows,
                    dy.as_mut_ptr(),
                    dy.len(),
                )
            };
            self.done(rc).then_some(dy)
        }

        fn moe_layer_q8_dev(
            &self,
            layer: usize,
            xs: &[f32],
            m: usize,
            plan: &[(usize, usize, usize)],
            slot_tok: &[i32],
            wslot: &[f32],
        ) -> Option<Vec<f32>> {
            let shape = *self.moe.get(&layer)?;
            if m == 0 || xs.len() != m * shape.hidden || slot_tok.len() != wslot.len() {
                return None;
            }
            let flat: Vec<usize> = plan.iter().flat_map(|&(e, off, cnt)| [e, off, cnt]).collect(); // (expert, slot_off, count)
            let mut y = vec![0f32; m * shape.hidden];
            let _g = self.lock.lock().unwrap();
            let rc = unsafe {
                ffi::smx_moe_layer(
                    self.ctx,
                    layer,
                    xs.as_ptr(),
                    m,
                    flat.as_ptr(),
                    plan.len(),
                    slot_tok.as_ptr(),
                    wslot.as_ptr(),
                    slot_tok.len(),
                    y.as_mut_ptr(),
                    y.len(),
                )
            };
            self.done(rc).then_some(y)
        }

        fn gemv(&self, key: &str, x: &[f32]) -> Option<Vec<f32>> {
            let k = cstr(key)?;
            let (_, out_dim) = self.dims(&k)?;
            let mut y = vec![0f32; out_dim];
            let _g = self.lock.lock().unwrap();
            // fp32 activations by default: the arithmetic of the kernels strix-backend-rocm launches for
            // `gemv` (decode.rs:3827-3898) and of the CPU path; `fast-gemv` opts into the decode path's
            // int8-activation GEMV (about 1e-2 relative from the CPU result).
            #[cfg(not(feature = "fast-gemv"))]
            let rc = unsafe { ffi::smx_gemv_f32(self.ctx, k.as_ptr(), x.as_ptr(), x.len(), y.as_mut_ptr(), y.len()) };
            #[cfg(feature = "fast-gemv")]
            let rc = unsafe { ffi::smx_gemv(self.ctx, k.as_ptr(), x.as_ptr(), x.len(), y.as_mut_ptr(), y.len()) };
            self.done(rc).then_some(y)
        }

        /// One device job and one sync for the whole batch (decode.rs:3227-3255), in the arithmetic
        /// of `gemv`: fp32 activations, one launch per item back to back; with `fast-gemv`
        /// consecutive items of one format and input length share a launch.
        fn gemv_batch(&self, calls: &[(&str, &[f32])]) -> Vec<Option<Vec<f32>>> {
            if calls.is_empty() {
                return Vec::new();
            }
            let n = calls.len();
            let keys: Vec<Option<CString>> = calls.iter().map(|(k, _)| cstr(k)).collect();
            // items whose key cannot be a C string or is not resident get a zero-length result
            // buffer and the library's status 0
            let empty = CString::new("").unwrap();
            let mut outs: Vec<Vec<f32>> = Vec::with_capacity(n);
            for k in &keys {
                let out_dim = k.as_ref().and_then(|k| self.dims(k)).map(|d| d.1).unwrap_or(0);
                outs.push(vec![0f32; out_dim]);
            }
            let key_ptrs: Vec<*const c_char> =
                keys.iter().map(|k| k.as_ref().unwrap_or(&empty).as_ptr()).collect();
            let x_ptrs: Vec<*const c_float> = calls.iter().map(|(_, x)| x.as_ptr()).collect();
            let in_lens: Vec<usize> = calls.iter().map(|(_, x)| x.len()).collect();
            let y_ptrs: Vec<*mut c_float> = outs.iter_mut().map(|y| y.as_mut_ptr()).collect();
            let out_caps: Vec<usize> = outs.iter().map(|y| y.len()).collect();
            let mut status = vec![0 as c_int; n];
            let rc = {
                let _g = self.lock.lock().unwrap();
                type BatchFn = unsafe extern "C" fn(
                    *mut ffi::SmxCtx,
                    usize,
                    *const *const c_char,
                    *const *const c_float,
                    *const usize,
                    *const *mut c_float,
                    *const usize,
                    *mut c_int,
                ) -> c_int;
                let batch: BatchFn =
                    if cfg!(feature = "fast-gemv") { ffi::smx_gemv_batch } else { ffi::smx_gemv_f32_batch };
                unsafe {
                    batch(
                        self.ctx,
                        n,
                        key_ptrs.as_ptr(),
                        x_ptrs.as_ptr(),
                        in_lens.as_ptr(),
                        y_ptrs.as_ptr(),
                        out_caps.as_ptr(),
                        status.as_mut_ptr(),
                    )
                }
            };
            if rc < 0 {
                tracing::warn!("mi355: {}", last_error(self.ctx));
            }
            outs.into_iter()
                .zip(status)
                .map(|(y, st)| (st == 1).then_some(y))
                .collect()
        }

        fn resident_count(&self) -> usize {
            unsafe { ffi::smx_resident_count(self.ctx) }
        }

        fn name(&self) -> &str {
            &self.name
        }
    }

    #[cfg(test)]
    mod tests {
        use super::*;

        fn f32_to_f16(v: f32) -> u16 {
            // positive normal values only (what the test generates)
            let bits = v.to_bits();
            let e = ((bits >> 23) & 0xff) as i32 - 127 + 15;
            let m = bits & 0x7f_ffff;
            let mut h = ((e as u32) << 10) | (m >> 13);
            if m & 0x1000 != 0 {
                h += 1; // round to nearest (ties away; the test data never lands on a tie)
            }
            h as u16
        }

        fn f16_to_f32(h: u16) -> f32 {
            let e = ((h >> 10) & 0x1f) as u32;
            let m = (h & 0x3ff) as u32;
            f32::from_bits(((e + 112) << 23) | (m << 13))
        }

        /// The device test of strix-backend-rocm (src/lib.rs:141-231) through the trait: the same
        /// generator, the same CPU sum, the same 1e-3 bar (the default build's fp32-activation `gemv`);
        /// the int8-activation `gemv` of a `fast-gemv` build is held to its own class (2e-2).
        #[test]
        #[ignore = "requires an MI355X"]
        fn mi355_q4_gemv_matches_cpu() {
            let (in_dim, out_dim) = (15360usize, 3840usize);
            let nblk = in_dim / 32;
            let total = nblk * out_dim;
            let mut raw = vec![0u8; total * 18];
            let mut seed = 0xA5A5_1234u64;
            let mut next = || {
                seed = seed.wrapping_mul(6364136223846793005).wrapping_add(1);
                (seed >> 33) as u32
            };
            for i in 0..total {
                let s = f32_to_f16(0.03 + (next() % 32) as f32 * 0.003);
                raw[i * 18..i * 18 + 2].copy_from_slice(&s.to_le_bytes());
                for w in 0..4 {
                    raw[i * 18 + 2 + w * 4..i * 18 + 6 + w * 4].copy_from_slice(&next().to_le_bytes());
                }
            }
            let x: Vec<f32> = (0..in_dim).map(|i| (i as f32 * 0.017).sin() * 0.5).collect();
            let cpu: Vec<f32> = (0..out_dim)
                .map(|row| {
                    let mut acc = 0.0f32;
                    for b in 0..nblk {
                        let blk = (row * nblk + b) * 18;
                        let d = f16_to_f32(u16::from_le_bytes([raw[blk], raw[blk + 1]]));
                        for j in 0..16 {
                            let byte = raw[blk + 2 + j];
                            let lo = (byte & 0xf) as f32 - 8.0;
                            let hi = (byte >> 4) as f32 - 8.0;
                            acc += d * (lo * x[b * 32 + j] + hi * x[b * 32 + j + 16]);
                        }
                    }
                    acc
                })
                .collect();
            let mut acc = Mi355WeightAccel::new().expect("MI355X device");
            assert!(acc.upload_q4_0("t.weight", &raw, in_dim, out_dim));
            let got = acc.gemv("t.weight", &x).expect("resident");
            let max_err = cpu.iter().zip(&got).map(|(c, g)| (c - g).abs()).fold(0.0f32, f32::max);
            let scale = cpu.iter().map(|v| v.abs()).fold(1e-6f32, f32::max);
            eprintln!("{}: rel_err {:.2e}", acc.name(), max_err / scale);
            let bar = if cfg!(feature = "fast-gemv") { 2e-2 } else { 1e-3 };
            assert!(max_err / scale < bar, "mi355 gemv diverged");
            assert!(acc.gemv("never.adopted", &x).is_none());
            assert_eq!(acc.resident_count(), 1);
        }
    }
}
