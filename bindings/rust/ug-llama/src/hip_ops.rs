//! `impl crate::Device for ug_hip::Device`: the five custom ops of ug-llama (src/main.rs:22-28) on
//! the MI355X backend, next to cpu_ops.rs, cuda_ops.rs and metal_ops.rs.
//!
//! Each op is an `LB::custom` closure (inputs first, the result last) around one entry point of
//! `libughip.so`; nothing is compiled at run time on this side.  Unlike the CUDA and Metal modules
//! (cuda_ops.rs:176-178, metal_ops.rs:179-181), `causal_mask` exists here, so prompts longer than
//! one token work on the device.
use crate::LB;
use ug::Result;
use ug_hip::ffi::{self, check};
use ug_hip::{Device, Slice};

fn rope_any(src: &LB<Device>, cos: &LB<Device>, sin: &LB<Device>, pos: &LB<Device>, interleaved: bool) -> Result<LB<Device>> {
    let (b, h, t, d) = src.shape().dims4()?;
    if src.dtype() != ug::DType::F32 {
        ug::bail!("rope: only f32 is supported, got {:?}", src.dtype())
    }
    let dev = src.device().clone();
    let f = move |vs: Vec<&mut Slice>| -> Result<()> {
        let [src, cos, sin, pos, dst]: [&mut Slice; 5] = match vs.try_into() {
            Ok(vs) => vs,
            Err(_) => ug::bail!("rope: expected 5 slices"),
        };
        check(unsafe {
            ffi::ughip_rope(dev.raw(), src.raw(), cos.raw(), sin.raw(), pos.raw(), dst.raw(), b * h, t, d, interleaved as std::ffi::c_int)
        })
    };
    LB::custom(f, vec![src.clone(), cos.clone(), sin.clone(), pos.clone()], (b, h, t, d), src.dtype(), src.device())
}

impl crate::Device for Device {
    fn rope_i(src: &LB<Self>, cos: &LB<Self>, sin: &LB<Self>, pos: &LB<Self>) -> Result<LB<Self>> {
        rope_any(src, cos, sin, pos, true)
    }

    fn rope(src: &LB<Self>, cos: &LB<Self>, sin: &LB<Self>, pos: &LB<Self>) -> Result<LB<Self>> {
        rope_any(src, cos, sin, pos, false)
    }

    fn cat(lhs: &LB<Self>, rhs: &LB<Self>, axis: usize) -> Result<LB<Self>> {
        let l_dims = lhs.dims();
        let r_dims = rhs.dims();
        if axis >= l_dims.len() {
            ug::bail!("unexpected axis {axis} for cat {l_dims:?}")
        }
        if l_dims.len() != r_dims.len() {
            ug::bail!("unexpected shapes for cat {l_dims:?} {r_dims:?} axis: {axis}")
        }
        for (i, (l, r)) in l_dims.iter().zip(r_dims.iter()).enumerate() {
            if axis != i && *l != *r {
                ug::bail!("unexpected shapes for cat {l_dims:?} {r_dims:?} axis: {axis}")
            }
        }
        let mut dst_dims = l_dims.to_vec();
        dst_dims[axis] = l_dims[axis] + r_dims[axis];
        let d1 = l_dims[..axis].iter().product::<usize>();
        let d2_l = l_dims[axis..].iter().product::<usize>();
        let d2_r = r_dims[axis..].iter().product::<usize>();
        let dev = lhs.device().clone();
        let f = move |vs: Vec<&mut Slice>| -> Result<()> {
            let [lhs, rhs, dst]: [&mut Slice; 3] = match vs.try_into() {
                Ok(vs) => vs,
                Err(_) => ug::bail!("cat: expected 3 slices"),
            };
            check(unsafe { ffi::ughip_cat(dev.raw(), lhs.raw(), rhs.raw(), dst.raw(), d1, d2_l, d2_r) })
        };
        LB::custom(f, vec![lhs.clone(), rhs.clone()], dst_dims, lhs.dtype(), lhs.device())
    }

    fn custom_softmax(src: &LB<Self>) -> Result<LB<Self>> {
        let rank = src.rank();
        let dim_m1 = src.dims()[rank - 1];
        let n_rows = src.shape().num_elements() / dim_m1;
        let dev = src.device().clone();
        let f = move |vs: Vec<&mut Slice>| -> Result<()> {
            let [src, dst]: [&mut Slice; 2] = match vs.try_into() {
                Ok(vs) => vs,
                Err(_) => ug::bail!("custom_softmax: expected 2 slices"),
            };
            check(unsafe { ffi::ughip_softmax_rows(dev.raw(), src.raw(), dst.raw(), n_rows, dim_m1) })
        };
        LB::custom(f, vec![src.clone()], src.shape(), src.dtype(), src.device())
    }

    fn causal_mask(src: &LB<Self>) -> Result<LB<Self>> {
        let (b, h, s1, s2) = src.shape().dims4()?;
        let dev = src.device().clone();
        let f = move |vs: Vec<&mut Slice>| -> Result<()> {
            let [src, dst]: [&mut Slice; 2] = match vs.try_into() {
                Ok(vs) => vs,
                Err(_) => ug::bail!("causal_mask: expected 2 slices"),
            };
            check(unsafe { ffi::ughip_causal_mask(dev.raw(), src.raw(), dst.raw(), b * h, s1, s2) })
        };
        LB::custom(f, vec![src.clone()], (b, h, s1, s2), src.dtype(), src.device())
    }
}

/// Opt-in fusions with no counterpart in the reference's trait: one launch for what model.rs:231-244
/// builds from several ops.  `Attention::fwd` can call these when the device is the HIP one.
pub mod fused {
    use super::*;

    /// `custom_softmax(causal_mask(att))` over `[b, h, s1, s2]`; masked entries are never read.
    pub fn causal_softmax(att: &LB<Device>) -> Result<LB<Device>> {
        let (b, h, s1, s2) = att.shape().dims4()?;
        let dev = att.device().clone();
        let f = move |vs: Vec<&mut Slice>| -> Result<()> {
            let [src, dst]: [&mut Slice; 2] = match vs.try_into() {
                Ok(vs) => vs,
                Err(_) => ug::bail!("causal_softmax: expected 2 slices"),
            };
            check(unsafe { ffi::ughip_causal_softmax_rows(dev.raw(), src.raw(), dst.raw(), b * h, s1, s2) })
        };
        LB::custom(f, vec![att.clone()], (b, h, s1, s2), att.dtype(), att.device())
    }

    /// One query position: q `[b, nh, 1, d]`, k and v `[b, nkv, s, d]` -> `[b, nh, 1, d]`
    /// (repeat, q k^T, scale, softmax, x v of model.rs:231-244 in one launch).
    pub fn attention_decode(q: &LB<Device>, k: &LB<Device>, v: &LB<Device>, scale: f32) -> Result<LB<Device>> {
        let (b, nh, t, d) = q.shape().dims4()?;
        let (_, nkv, s, _) = k.shape().dims4()?;
        if t != 1 {
            ug::bail!("attention_decode: one query position expected, got {t}")
        }
        let dev = q.device().clone();
        let f = move |vs: Vec<&mut Slice>| -> Result<()> {
            let [q, k, v, dst]: [&mut Slice; 4] = match vs.try_into() {
                Ok(vs) => vs,
                Err(_) => ug::bail!("attention_decode: expected 4 slices"),
            };
            check(unsafe { ffi::ughip_attention_decode(dev.raw(), q.raw(), k.raw(), v.raw(), dst.raw(), b, nh, nkv, s, d, scale) })
        };
        LB::custom(f, vec![q.clone(), k.clone(), v.clone()], (b, nh, 1, d), q.dtype(), q.device())
    }
}
