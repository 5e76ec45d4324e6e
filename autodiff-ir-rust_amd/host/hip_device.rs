//! `HipDevice`: the MI355X backend behind the crate's `Device` trait (reference src/core/ir.rs:126-143), over the C ABI
//! of include/adhip.h.  To be placed at `src/devices/hip/mod.rs` of the reference crate (with `pub mod hip;` in
//! `src/devices/mod.rs`) and linked with `-ladhip`.
//!
//! NOT COMPILED IN THIS REPOSITORY: the build image has no Rust toolchain.  What keeps this file honest without one:
//!   * `serialize` below writes the wire format field by field in the order of `enum IRCmds`
//!     (reference src/core/ir.rs:8-105); the same format is written by adhip/ir.py and host/adhip_device.hpp, which
//!     tests/test_wire_format.py holds to the committed bytes of tests/golden/wire_every_command.bin.  The unit test
//!     at the bottom of this file builds that same program and compares with those bytes, for whoever builds it.
//!   * the FFI declarations are the prototypes of include/adhip.h, one for one.
//!
//! How it fits the trait.  `Device::execute` receives the crate's own lowering (`KernelProcedure`), which this device
//! does not use: it lowers the IR itself, behind the C ABI.  `ir_callback` runs after `EX` has been appended and before
//! anything else (reference src/core/autodiff.rs:108-114), sees the complete IR and keeps a copy; `execute` serialises
//! that copy.  The crate calls `to_kernel` before `execute` (src/core/ir.rs:180-198); it panics on `Index` and cannot
//! express `Concat` for its device, so programs that use them need `ir_b_execute` to skip `to_kernel` for a device that
//! lowers by itself (one `if` around that call, keyed on a new defaulted trait method such as `lowers_ir() -> bool`).

use std::cell::RefCell;
use std::ffi::{c_char, c_int, c_void, CStr, CString};
use std::sync::Arc;

use crate::core::dependency::ret_dep_list;
use crate::kernel_decl::KernelProcedure;
use crate::trackers::KernelTracker;
use crate::{Device, IRBase, IRCmds, IRProcedure, ValueData};

#[link(name = "adhip")]
extern "C" {
    fn adhip_create(device_ordinal: c_int, out: *mut *mut c_void) -> c_int;
    fn adhip_destroy(ctx: *mut c_void);
    fn adhip_last_error(ctx: *mut c_void) -> *const c_char;
    fn adhip_execute(ctx: *mut c_void, program: *const u8, program_len: usize, dep_ids: *const *const c_char,
                     n_dep_ids: usize) -> c_int;
    fn adhip_get_tensor(ctx: *mut c_void, id: *const c_char, data: *mut *const f32, dims: *mut *const u64,
                        ndim: *mut usize) -> c_int;
    fn adhip_dot_prod_shape(a_dims: *const u64, a_ndim: usize, b_dims: *const u64, b_ndim: usize, out: *mut u64) -> c_int;
}

// ---------------------------------------------------------------------------------------------------------------
// wire format (little-endian):
//   stream := "ADIR" u32(1) proc          proc := str(id) u32(ncmds) cmd*          str := u32(len) bytes
//   dims   := u32(n) u64*n                cmd  := u8(tag) fields, tag = position of the variant in `enum IRCmds`
// ---------------------------------------------------------------------------------------------------------------

fn put_u32(o: &mut Vec<u8>, v: u32) { o.extend_from_slice(&v.to_le_bytes()); }
fn put_u64(o: &mut Vec<u8>, v: u64) { o.extend_from_slice(&v.to_le_bytes()); }
fn put_f32(o: &mut Vec<u8>, v: f32) { o.extend_from_slice(&v.to_le_bytes()); }
fn put_str(o: &mut Vec<u8>, s: &str) { put_u32(o, s.len() as u32); o.extend_from_slice(s.as_bytes()); }
fn put_dims(o: &mut Vec<u8>, d: &[usize]) { put_u32(o, d.len() as u32); for &x in d { put_u64(o, x as u64); } }

fn put_proc(o: &mut Vec<u8>, p: &IRProcedure, payload_offsets: &mut Vec<usize>) {
    put_str(o, &p.id);
    put_u32(o, p.main.len() as u32);
    for cmd in &p.main {
        match cmd {
            IRCmds::CreateMat { contents, dim, id } => {
                o.push(0);
                put_str(o, id);
                put_dims(o, dim);
                payload_offsets.push(o.len());
                // borrowed until adhip_execute returns: the IR is locked for the whole call (src/core/ir.rs:182-186)
                put_u64(o, if contents.is_empty() { 0 } else { contents.as_ptr() as u64 });
                put_u64(o, contents.len() as u64);
            }
            IRCmds::CreateConstant { contents, id, dim } => { o.push(1); put_f32(o, *contents); put_str(o, id); put_dims(o, dim); }
            IRCmds::ElwMultiply { a, b, res } => { o.push(2); put_str(o, a); put_str(o, b); put_str(o, res); }
            IRCmds::ElwAdd { a, b, res } => { o.push(3); put_str(o, a); put_str(o, b); put_str(o, res); }
            IRCmds::ElwMultiplyEq { s, o: other } => { o.push(4); put_str(o, s); put_str(o, other); }
            IRCmds::ElwAddEq { s, o: other } => { o.push(5); put_str(o, s); put_str(o, other); }
            IRCmds::EqualZero { a, res } => { o.push(6); put_str(o, a); put_str(o, res); }
            IRCmds::MoreZero { a, res } => { o.push(7); put_str(o, a); put_str(o, res); }
            IRCmds::LessZero { a, res } => { o.push(8); put_str(o, a); put_str(o, res); }
            IRCmds::Sum { a, res } => { o.push(9); put_str(o, a); put_str(o, res); }
            IRCmds::DotProduct { a, b, res } => { o.push(10); put_str(o, a); put_str(o, b); put_str(o, res); }
            IRCmds::View { a, target_dim, res } => { o.push(11); put_str(o, a); put_dims(o, target_dim); put_str(o, res); }
            IRCmds::Index { a, index, dim, res } => { o.push(12); put_str(o, a); put_u64(o, *index as u64); put_u64(o, *dim as u64); put_str(o, res); }
            IRCmds::Concat { a, b, dim, res } => { o.push(13); put_str(o, a); put_str(o, b); put_u64(o, *dim as u64); put_str(o, res); }
            IRCmds::Permute { a, p, res } => { o.push(14); put_str(o, a); put_dims(o, p); put_str(o, res); }
            IRCmds::Broadcast { a, dim, r, res } => { o.push(15); put_str(o, a); put_u64(o, *dim as u64); put_u64(o, *r as u64); put_str(o, res); }
            IRCmds::Contigious { a, res } => { o.push(16); put_str(o, a); put_str(o, res); }
            IRCmds::Exp2 { a, res } => { o.push(17); put_str(o, a); put_str(o, res); }
            IRCmds::Log2 { a, res } => { o.push(18); put_str(o, a); put_str(o, res); }
            IRCmds::Sin { a, res } => { o.push(19); put_str(o, a); put_str(o, res); }
            IRCmds::Recip { a, res } => { o.push(20); put_str(o, a); put_str(o, res); }
            IRCmds::Sqrt { a, res } => { o.push(21); put_str(o, a); put_str(o, res); }
            IRCmds::While { conditional_var, block } => { o.push(22); put_str(o, conditional_var); put_proc(o, block, payload_offsets); }
            IRCmds::If { conditions, else_proc } => {
                o.push(23);
                put_u32(o, conditions.len() as u32);
                for (cond, block) in conditions { put_str(o, cond); put_proc(o, block, payload_offsets); }
                match else_proc {
                    Some(block) => { o.push(1); put_proc(o, block, payload_offsets); }
                    None => o.push(0),
                }
            }
            IRCmds::EX => o.push(24),
            IRCmds::Heading { cmt } => { o.push(25); put_str(o, cmt); }
            // The library also accepts tag 26, `Max {a, res}` (fields as Sum): the row maximum the crate declares as
            // `ReduceOp::Max` (src/kernel/kernel_decl.rs:75-78) and lists as to-do in src/core/ir.rs:49.  Once
            // `IRCmds` has that variant:
            // IRCmds::Max { a, res } => { o.push(26); put_str(o, a); put_str(o, res); }
        }
    }
}

/// The program as adhip_execute reads it, and the byte offsets of the CreateMat pointer fields inside it.
pub fn serialize(proc: &IRProcedure) -> (Vec<u8>, Vec<usize>) {
    let mut o = Vec::with_capacity(4096);
    let mut payload_offsets = Vec::new();
    o.extend_from_slice(b"ADIR");
    put_u32(&mut o, 1);
    put_proc(&mut o, proc, &mut payload_offsets);
    (o, payload_offsets)
}

// ---------------------------------------------------------------------------------------------------------------

pub struct HipDevice {
    ctx: *mut c_void,
    captured: RefCell<Option<IRProcedure>>, // ir_callback takes &self
}

// every call into the device is made under the crate's DEVICE mutex (src/core/ir.rs:180-186, src/core/value.rs:83-91)
unsafe impl Send for HipDevice {}
unsafe impl Sync for HipDevice {}

impl HipDevice {
    pub fn new(device_ordinal: i32) -> HipDevice {
        let mut ctx: *mut c_void = std::ptr::null_mut();
        let rc = unsafe { adhip_create(device_ordinal as c_int, &mut ctx) };
        if rc != 0 || ctx.is_null() {
            panic!("adhip_create failed: {}", Self::error_text(std::ptr::null_mut()));
        }
        HipDevice { ctx, captured: RefCell::new(None) }
    }

    fn error_text(ctx: *mut c_void) -> String {
        let p = unsafe { adhip_last_error(ctx) };
        if p.is_null() { String::new() } else { unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned() }
    }
}

impl Device for HipDevice {
    fn ir_callback(&self, irb: &mut IRBase) {
        *self.captured.borrow_mut() = Some(irb.proc.clone()); // CreateMat contents are Arc: no payload is copied
    }

    fn execute(&mut self, _proc: KernelProcedure, _tracker: KernelTracker) {
        let proc = self.captured.borrow_mut().take().expect("HipDevice::execute without a preceding ir_callback");
        let (blob, _) = serialize(&proc);
        let deps: Vec<CString> = ret_dep_list().into_iter().filter(|s| !s.is_empty()).map(|s| CString::new(s).unwrap()).collect();
        let ptrs: Vec<*const c_char> = deps.iter().map(|s| s.as_ptr()).collect();
        let rc = unsafe { adhip_execute(self.ctx, blob.as_ptr(), blob.len(), ptrs.as_ptr(), ptrs.len()) };
        drop(proc); // the payload pointers inside `blob` were valid until here
        if rc != 0 {
            panic!("adhip_execute failed: {}", Self::error_text(self.ctx)); // the reference's devices panic too
        }
    }

    fn get_tensor(&self, id: &String) -> ValueData {
        let cid = CString::new(id.as_str()).unwrap();
        let mut data: *const f32 = std::ptr::null();
        let mut dims: *const u64 = std::ptr::null();
        let mut ndim: usize = 0;
        match unsafe { adhip_get_tensor(self.ctx, cid.as_ptr(), &mut data, &mut dims, &mut ndim) } {
            0 => {
                let dim: Vec<usize> = unsafe { std::slice::from_raw_parts(dims, ndim) }.iter().map(|&d| d as usize).collect();
                let n: usize = dim.iter().product();
                // the context owns the memory (valid until the next execute): copy it out
                let values = if n == 0 { Vec::new() } else { unsafe { std::slice::from_raw_parts(data, n) }.to_vec() };
                ValueData { dim, data: Arc::new(values), id: id.clone(), is_none: false }
            }
            1 => ValueData::none(),
            _ => panic!("adhip_get_tensor failed: {}", Self::error_text(self.ctx)),
        }
    }

    fn dot_prod_shape(&self, a: &Vec<usize>, b: &Vec<usize>) -> Vec<usize> {
        let a64: Vec<u64> = a.iter().map(|&x| x as u64).collect();
        let b64: Vec<u64> = b.iter().map(|&x| x as u64).collect();
        let mut out = [0u64; 2];
        let rc = unsafe { adhip_dot_prod_shape(a64.as_ptr(), a64.len(), b64.as_ptr(), b64.len(), out.as_mut_ptr()) };
        assert_eq!(rc, 0, "dot_prod_shape of an empty shape");
        vec![out[0] as usize, out[1] as usize]
    }
}

impl Drop for HipDevice {
    fn drop(&mut self) {
        unsafe { adhip_destroy(self.ctx) }
    }
}

#[cfg(test)]
mod tests {
    use super::*;
    use crate::IRCmds::*;

    fn s(x: &str) -> String { x.to_string() }

    /// The program of tests/golden/make_wire_fixture.py without its last-but-one command (Max, which `IRCmds` does
    /// not have): the bytes must equal tests/golden/wire_every_command.bin with that command cut out, i.e. with the
    /// command count 33 instead of 34 and the 12 bytes `1a 01000000 'e' 02000000 'm' 'x'` before the final `18` removed
    /// (tests/test_wire_format.py checks that this edit of the fixture is what a writer without Max produces).
    #[test]
    fn wire_format_matches_the_fixture() {
        let proc_of = |id: &str, main: Vec<IRCmds>| IRProcedure { main, id: s(id) };
        let body = proc_of("loop", vec![ElwAddEq { s: s("k"), o: s("m1") }, MoreZero { a: s("k"), res: s("cond") }]);
        let arm0 = proc_of("arm0", vec![ElwMultiplyEq { s: s("e"), o: s("c") }]);
        let arm1 = proc_of("arm1", vec![CreateConstant { contents: 2.0, id: s("two"), dim: vec![2, 3] }, ElwAddEq { s: s("e"), o: s("two") }]);
        let other = proc_of("other", vec![Heading { cmt: s("neither predicate held") }]);
        let main = proc_of("main", vec![
            Heading { cmt: s("every command once") },
            CreateMat { contents: Arc::new(vec![1., 2., 3., 4., 5., 6.]), dim: vec![2, 3], id: s("a") },
            CreateMat { contents: Arc::new(vec![1., 0., -1., 2., 0.5, 4.]), dim: vec![3, 2], id: s("b") },
            CreateConstant { contents: 0.5, id: s("c"), dim: vec![2, 3] },
            ElwMultiply { a: s("a"), b: s("c"), res: s("d") },
            ElwAdd { a: s("a"), b: s("d"), res: s("e") },
            ElwMultiplyEq { s: s("e"), o: s("c") },
            ElwAddEq { s: s("e"), o: s("a") },
            EqualZero { a: s("e"), res: s("f") },
            MoreZero { a: s("e"), res: s("g") },
            LessZero { a: s("e"), res: s("h") },
            Sum { a: s("e"), res: s("s") },
            DotProduct { a: s("a"), b: s("b"), res: s("p") },
            View { a: s("a"), target_dim: vec![3, 2], res: s("v") },
            Index { a: s("a"), index: 1, dim: 0, res: s("i") },
            Concat { a: s("a"), b: s("a"), dim: 0, res: s("cc") },
            Permute { a: s("a"), p: vec![1, 0], res: s("t") },
            View { a: s("s"), target_dim: vec![2, 1], res: s("s1") },
            Broadcast { a: s("s1"), dim: 1, r: 3, res: s("sb") },
            Contigious { a: s("t"), res: s("tc") },
            Exp2 { a: s("a"), res: s("x2") },
            Log2 { a: s("x2"), res: s("l2") },
            Sin { a: s("a"), res: s("sn") },
            Recip { a: s("x2"), res: s("rc") },
            Sqrt { a: s("x2"), res: s("sq") },
            CreateMat { contents: Arc::new(vec![2.]), dim: vec![1], id: s("k") },
            CreateConstant { contents: -1.0, id: s("m1"), dim: vec![1] },
            MoreZero { a: s("k"), res: s("cond") },
            While { conditional_var: s("cond"), block: body },
            EqualZero { a: s("k"), res: s("is0") },
            LessZero { a: s("k"), res: s("neg") },
            If { conditions: vec![(s("neg"), arm0), (s("is0"), arm1)], else_proc: Some(other) },
            EX,
        ]);
        let (mut blob, offsets) = serialize(&main);
        for o in offsets { for i in 0..8 { blob[o + i] = 0; } }
        let mut want = std::fs::read("tests/golden/wire_every_command.bin").expect("fixture of the adhip repository");
        // cut the Max command (tag 26, str("e"), str("mx") = 12 bytes) that sits before the final EX byte
        let cut = want.len() - 1 - 12;
        assert_eq!(want[cut], 26u8);
        want.drain(cut..cut + 12);
        let count_at = 8 + 4 + 4; // magic and version, then str("main")
        want[count_at..count_at + 4].copy_from_slice(&33u32.to_le_bytes());
        assert_eq!(blob, want);
    }
}
