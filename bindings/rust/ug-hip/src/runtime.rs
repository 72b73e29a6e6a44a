//! `ug::Device` / `ug::Slice` for one MI355X behind `libughip.so`.
//!
//! What `ug-cuda/src/runtime.rs:80-393` is for CUDA.  Handles are reference-counted by the
//! library: cloning a `Device` retains it, dropping releases it; a `Slice` owns its allocation
//! and a `Func` its compiled kernel.  The one part with any content on this side is the
//! serialiser that turns an `ssa::Kernel` into the flat POD image `ughip_compile` takes.
use crate::ffi::{self, check, UghipA, UghipInstr, UghipKernelArg, UghipSsa};
use std::ffi::{c_int, c_void, CString};
use ug::lang::ssa;
use ug::{DType, Layout, Result, WithDType};

/// `UGHIP_*` code of a dtype: BF16 = 0, F16 = 1, F32 = 2, I32 = 3, I64 = 4.
fn dtype_code(dtype: DType) -> c_int {
    match dtype {
        DType::BF16 => ffi::UGHIP_BF16,
        DType::F16 => ffi::UGHIP_F16,
        DType::F32 => ffi::UGHIP_F32,
        DType::I32 => ffi::UGHIP_I32,
        DType::I64 => ffi::UGHIP_I64,
    }
}

fn dtype_of_code(code: c_int) -> Result<DType> {
    let dtype = match code {
        ffi::UGHIP_BF16 => DType::BF16,
        ffi::UGHIP_F16 => DType::F16,
        ffi::UGHIP_F32 => DType::F32,
        ffi::UGHIP_I32 => DType::I32,
        ffi::UGHIP_I64 => DType::I64,
        _ => ug::bail!("unknown dtype code {code} from libughip"),
    };
    Ok(dtype)
}

pub struct Device {
    raw: *mut ffi::UghipDevice,
}

impl Device {
    /// `Device::new(ordinal)` (ug-cuda/src/runtime.rs:158-177).
    pub fn new(ordinal: usize) -> Result<Self> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::ughip_device_create(ordinal as c_int, &mut raw) })?;
        Ok(Self { raw })
    }

    pub fn raw(&self) -> *mut ffi::UghipDevice {
        self.raw
    }

    /// Fresh allocations are zero-filled by default, like the CPU backend's (cpu_runtime.rs:255-264);
    /// `false` gives ug-cuda's truly uninitialised memory and saves a fill per allocation.
    pub fn set_zero_fill(&self, on: bool) -> Result<()> {
        check(unsafe { ffi::ughip_device_set_zero_fill(self.raw, on as c_int) })
    }

    /// The architecture the library compiles for, e.g. "gfx950".
    pub fn arch(&self) -> Result<String> {
        let mut buf = [0 as std::ffi::c_char; 64];
        check(unsafe { ffi::ughip_device_arch(self.raw, buf.as_mut_ptr(), buf.len()) })?;
        Ok(unsafe { std::ffi::CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned())
    }

    /// HIP source built with hiprtc, kernel `entry` launched with a fixed configuration: the
    /// counterpart of `compile_cu` (ug-cuda/src/runtime.rs:179-186).
    pub fn compile_hip(
        &self,
        source: &str,
        entry: &str,
        arg_dtypes: &[DType],
        cfg: ug::lang::LaunchConfig,
    ) -> Result<Func> {
        let source = CString::new(source).map_err(ug::Error::msg)?;
        let entry = CString::new(entry).map_err(ug::Error::msg)?;
        let codes: Vec<c_int> = arg_dtypes.iter().map(|d| dtype_code(*d)).collect();
        let mut raw = std::ptr::null_mut();
        check(unsafe {
            ffi::ughip_compile_source(
                self.raw,
                source.as_ptr(),
                entry.as_ptr(),
                codes.len(),
                codes.as_ptr(),
                cfg.grid_dim,
                cfg.block_dim,
                cfg.shared_mem,
                &mut raw,
            )
        })?;
        Ok(Func { raw })
    }

    /// `Device::slice_from_values` of the other backends: allocate and upload.
    pub fn slice_from_values<DT: WithDType>(&self, vs: &[DT]) -> Result<Slice> {
        use ug::{Device as D, Slice as S};
        let mut slice = unsafe { self.allocate_uninit(DT::DTYPE, vs.len())? };
        slice.copy_host_to_device(vs)?;
        Ok(slice)
    }
}

impl Clone for Device {
    fn clone(&self) -> Self {
        // retain cannot fail for a live handle
        unsafe { ffi::ughip_device_retain(self.raw) };
        Self { raw: self.raw }
    }
}

impl Drop for Device {
    fn drop(&mut self) {
        unsafe { ffi::ughip_device_release(self.raw) };
    }
}

impl std::fmt::Debug for Device {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "HipDevice({:p})", self.raw)
    }
}

pub struct Slice {
    raw: *mut ffi::UghipSlice,
    len: usize,
    dtype: DType,
    device: Device,
}

impl Slice {
    pub fn raw(&self) -> *mut ffi::UghipSlice {
        self.raw
    }
}

impl Drop for Slice {
    fn drop(&mut self) {
        // goes back to the device's pool; the stream orders its reuse behind the work queued so far
        unsafe { ffi::ughip_free(self.raw) };
    }
}

impl std::fmt::Debug for Slice {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "HipSlice({:?}, len {})", self.dtype, self.len)
    }
}

impl ug::Slice for Slice {
    type Device = Device;

    fn device(&self) -> &Device {
        &self.device
    }

    fn dtype(&self) -> DType {
        self.dtype
    }

    fn len(&self) -> usize {
        self.len
    }

    fn copy_host_to_device<DT: WithDType>(&mut self, src: &[DT]) -> Result<()> {
        // the library checks length and dtype and words the errors like cpu_runtime.rs:376-391
        check(unsafe { ffi::ughip_h2d(self.raw, src.as_ptr() as *const c_void, dtype_code(DT::DTYPE), src.len()) })
    }

    fn copy_device_to_host<DT: WithDType>(&self, dst: &mut [DT]) -> Result<()> {
        check(unsafe { ffi::ughip_d2h(self.raw, dst.as_mut_ptr() as *mut c_void, dtype_code(DT::DTYPE), dst.len()) })
    }
}

pub struct Func {
    raw: *mut ffi::UghipFunc,
}

impl Func {
    pub fn raw(&self) -> *mut ffi::UghipFunc {
        self.raw
    }

    /// The HIP source the kernel was lowered to (what `Kernel.cuda_code()` is for ug-cuda).
    pub fn source(&self) -> String {
        let n = unsafe { ffi::ughip_func_source(self.raw, std::ptr::null_mut(), 0) };
        let mut buf = vec![0u8; n + 1];
        unsafe { ffi::ughip_func_source(self.raw, buf.as_mut_ptr() as *mut std::ffi::c_char, buf.len()) };
        buf.truncate(n);
        String::from_utf8_lossy(&buf).into_owned()
    }

    pub fn info(&self) -> Result<ffi::UghipFuncInfo> {
        let mut info = ffi::UghipFuncInfo::default();
        check(unsafe { ffi::ughip_func_get_info(self.raw, &mut info) })?;
        Ok(info)
    }
}

impl Drop for Func {
    fn drop(&mut self) {
        unsafe { ffi::ughip_func_release(self.raw) };
    }
}

// ---- ssa::Kernel -> ughip_ssa ------------------------------------------------------------------

fn wire_const(c: &ug::Const) -> UghipA {
    // 16-bit floats travel widened to f32, which is exact
    let z = UghipA { is_const: 1, ..Default::default() };
    match *c {
        ug::Const::I32(v) => UghipA { dtype: ffi::UGHIP_I32 as u8, i: v as i64, ..z },
        ug::Const::I64(v) => UghipA { dtype: ffi::UGHIP_I64 as u8, i: v, ..z },
        ug::Const::BF16(v) => UghipA { dtype: ffi::UGHIP_BF16 as u8, f: v.to_f32(), ..z },
        ug::Const::F16(v) => UghipA { dtype: ffi::UGHIP_F16 as u8, f: v.to_f32(), ..z },
        ug::Const::F32(v) => UghipA { dtype: ffi::UGHIP_F32 as u8, f: *v, ..z },
    }
}

fn wire_a(a: &ssa::A) -> UghipA {
    match a {
        ssa::A::Var(v) => UghipA { var: v.as_usize() as u32, ..Default::default() },
        ssa::A::Const(c) => wire_const(c),
    }
}

/// `UGHIP_U_*`: Id 0, Exp 1, Sin 2, Cos 3, Neg 4, Sqrt 5, Cast 6 (the target type is the
/// instruction's dtype).
fn unary_code(op: &ug::lang::UnaryOp) -> i32 {
    use ug::lang::UnaryOp::*;
    match op {
        Id => 0,
        Exp => 1,
        Sin => 2,
        Cos => 3,
        Neg => 4,
        Sqrt => 5,
        Cast(_) => 6,
    }
}

/// `UGHIP_B_*`, the order of `BinaryOp` (ug-core/src/lang.rs:24-32).
fn binary_code(op: &ug::lang::BinaryOp) -> i32 {
    use ug::lang::BinaryOp::*;
    match op {
        Add => 0,
        Sub => 1,
        Mul => 2,
        Div => 3,
        Mod => 4,
        Min => 5,
        Max => 6,
    }
}

/// `UGHIP_R_*`, the order of `ReduceOp` (ug-core/src/lang.rs:5-10).
fn reduce_code(op: &ug::lang::ReduceOp) -> i32 {
    use ug::lang::ReduceOp::*;
    match op {
        Sum => 0,
        Max => 1,
        Min => 2,
    }
}

fn wire_instr(instr: &ssa::Instr) -> UghipInstr {
    use ssa::Instr::*;
    let z = UghipInstr::default();
    // `op` is the discriminant in declaration order (ug-core/src/lang.rs:690-709)
    match instr {
        DefineAcc(c) => UghipInstr { op: 0, dtype: dtype_code(c.dtype()), a: wire_const(c), ..z },
        DefineGlobal { index, dtype } => UghipInstr { op: 1, dtype: dtype_code(*dtype), n: *index as u64, ..z },
        DefineLocal { size, dtype } => UghipInstr { op: 2, dtype: dtype_code(*dtype), n: *size as u64, ..z },
        Special(s) => {
            let sub = match s {
                ssa::Special::ThreadIdx => 0,
                ssa::Special::BlockIdx => 1,
            };
            UghipInstr { op: 3, dtype: ffi::UGHIP_I32, sub, ..z }
        }
        Const(c) => UghipInstr { op: 4, dtype: dtype_code(c.dtype()), a: wire_const(c), ..z },
        Unary { op, arg, dtype } => UghipInstr { op: 5, sub: unary_code(op), dtype: dtype_code(*dtype), a: wire_a(arg), ..z },
        Binary { op, lhs, rhs, dtype } => {
            UghipInstr { op: 6, sub: binary_code(op), dtype: dtype_code(*dtype), a: wire_a(lhs), b: wire_a(rhs), ..z }
        }
        Range { lo, up, step, end_idx } => {
            UghipInstr { op: 7, dtype: ffi::UGHIP_I32, a: wire_a(lo), b: wire_a(up), n: *step as u64, v: end_idx.as_usize() as u32, ..z }
        }
        Load { src, offset, dtype } => UghipInstr { op: 8, v: src.as_usize() as u32, a: wire_a(offset), dtype: dtype_code(*dtype), ..z },
        Assign { dst, src } => UghipInstr { op: 9, v: dst.as_usize() as u32, a: wire_a(src), ..z },
        EndRange { start_idx } => UghipInstr { op: 10, v: start_idx.as_usize() as u32, ..z },
        If { cond, end_idx } => UghipInstr { op: 11, a: wire_a(cond), v: end_idx.as_usize() as u32, ..z },
        EndIf => UghipInstr { op: 12, ..z },
        Store { dst, offset, value, dtype } => {
            UghipInstr { op: 13, v: dst.as_usize() as u32, a: wire_a(offset), b: wire_a(value), dtype: dtype_code(*dtype), ..z }
        }
        Barrier => UghipInstr { op: 14, ..z },
        ReduceLocal { op, arg, dtype } => UghipInstr { op: 15, sub: reduce_code(op), a: wire_a(arg), dtype: dtype_code(*dtype), ..z },
    }
}

/// The POD image of a kernel together with the vectors its pointers name.
struct Wire {
    instrs: Vec<UghipInstr>,
    args: Vec<UghipKernelArg>,
    launch: ug::lang::LaunchConfig,
}

impl Wire {
    fn new(kernel: &ssa::Kernel) -> Result<Self> {
        let instrs = kernel.instrs().iter().map(wire_instr).collect();
        let mut args = Vec::with_capacity(kernel.args().len());
        for (arg, line_no) in kernel.args().iter() {
            let (is_ptr, dtype) = match arg.type_() {
                ug::lang::Type::Ptr(dtype) => (1u8, dtype),
                // only pointer arguments are supported, as in lower_op.rs:413-416 and both GPU backends
                ug::lang::Type::Value(dtype) => (0u8, dtype),
            };
            args.push(UghipKernelArg {
                arg_id: arg.id().as_usize() as u64,
                is_ptr,
                dtype: dtype_code(dtype) as u8,
                pad_: 0,
                var: *line_no as u32,
            });
        }
        Ok(Self { instrs, args, launch: *kernel.launch_config() })
    }

    fn ssa(&self) -> UghipSsa {
        UghipSsa {
            instrs: self.instrs.as_ptr(),
            n_instrs: self.instrs.len(),
            args: self.args.as_ptr(),
            n_args: self.args.len(),
            grid_dim: self.launch.grid_dim,
            block_dim: self.launch.block_dim,
            shared_mem: self.launch.shared_mem,
            pad_: 0,
        }
    }
}

/// HIP source for a kernel without a device: what `code_gen::gen` is for ug-cuda
/// (ug-cuda/src/code_gen.rs:68-186), statement by statement for the kernel's own launch shape.
pub fn hip_code(kernel: &ssa::Kernel, name: &str) -> Result<String> {
    let wire = Wire::new(kernel)?;
    let ssa = wire.ssa();
    let name = CString::new(name).map_err(ug::Error::msg)?;
    let mut len = 0usize;
    check(unsafe { ffi::ughip_codegen_as_written(&ssa, name.as_ptr(), std::ptr::null_mut(), 0, &mut len) })?;
    let mut buf = vec![0u8; len + 1];
    check(unsafe { ffi::ughip_codegen_as_written(&ssa, name.as_ptr(), buf.as_mut_ptr() as *mut std::ffi::c_char, buf.len(), &mut len) })?;
    buf.truncate(len);
    Ok(String::from_utf8_lossy(&buf).into_owned())
}

impl ug::Device for Device {
    type Slice = Slice;
    type Func = Func;

    unsafe fn allocate_uninit(&self, dtype: DType, len: usize) -> Result<Slice> {
        let mut raw = std::ptr::null_mut();
        check(ffi::ughip_alloc(self.raw, dtype_code(dtype), len, &mut raw))?;
        // what the library recorded, not what was asked for: a mismatch would be a bug worth hearing about
        let got = dtype_of_code(ffi::ughip_slice_dtype(raw))?;
        let got_len = ffi::ughip_slice_len(raw);
        if got != dtype || got_len != len {
            ffi::ughip_free(raw);
            ug::bail!("ughip_alloc returned {got:?} x {got_len} for {dtype:?} x {len}")
        }
        Ok(Slice { raw, len, dtype, device: self.clone() })
    }

    fn synchronize(&self) -> Result<()> {
        check(unsafe { ffi::ughip_synchronize(self.raw) })
    }

    fn compile(&self, kernel: &ssa::Kernel, name: Option<&str>) -> Result<Func> {
        let wire = Wire::new(kernel)?;
        let ssa = wire.ssa();
        // the library sanitises and uniquifies the name itself (ug-cuda/src/runtime.rs:249-253 does it here)
        let name = match name {
            Some(name) => Some(CString::new(name).map_err(ug::Error::msg)?),
            None => None,
        };
        let name_ptr = name.as_ref().map_or(std::ptr::null(), |n| n.as_ptr());
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::ughip_compile(self.raw, &ssa, name_ptr, &mut raw) })?;
        Ok(Func { raw })
    }

    fn run(&self, f: &Func, args: &mut [&mut Slice]) -> Result<()> {
        // any number of arguments; asynchronous like ug-cuda's (runtime.rs:266-332); the library checks
        // dtypes, lengths against the offsets the kernel can form, and aliasing
        let ptrs: Vec<*mut ffi::UghipSlice> = args.iter().map(|s| s.raw).collect();
        check(unsafe { ffi::ughip_run(self.raw, f.raw, ptrs.as_ptr(), ptrs.len()) })
    }

    fn matmul(
        &self,
        dst: &mut Slice,
        lhs: &Slice,
        rhs: &Slice,
        bmnk: (usize, usize, usize, usize),
        lhs_l: &Layout,
        rhs_l: &Layout,
    ) -> Result<()> {
        let (b, m, n, k) = bmnk;
        if lhs_l.rank() != rhs_l.rank() {
            ug::bail!("matmul: layouts of different ranks {lhs_l:?} {rhs_l:?}")
        }
        check(unsafe {
            ffi::ughip_matmul(
                self.raw,
                dst.raw,
                lhs.raw,
                rhs.raw,
                b,
                m,
                n,
                k,
                lhs_l.rank(),
                lhs_l.dims().as_ptr(),
                lhs_l.strides().as_ptr(),
                lhs_l.offset(),
                rhs_l.dims().as_ptr(),
                rhs_l.strides().as_ptr(),
                rhs_l.offset(),
            )
        })
    }

    /// The backend asks for the serial loop nest (the SSA the CPU backend gets) and maps it to
    /// workgroups, waves and lanes itself: the scheduler's grid heuristic (schedule.rs:162-188)
    /// hard-codes 32-thread blocks.
    fn use_grid() -> bool {
        false
    }
}
