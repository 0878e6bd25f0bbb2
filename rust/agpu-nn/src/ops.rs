//! nn::ops: free functions `ops::*(…, &Arc<KernelRegistry>) -> Result<GpuTensor>` (nn/ops/mod.rs:19-37).  Shape checks
//! happen here, before the launch, as in the reference; outputs are allocated and returned.
use std::sync::Arc;

use agpu_sys as sys;

use crate::error::{NnError, Result};
use crate::registry::KernelRegistry;
use crate::tensor::GpuTensor;

fn mismatch(expected: String, actual: String) -> NnError {
    NnError::ShapeMismatch { expected, actual }
}

/// ops::layer_norm (nn/ops/norm.rs:14-81).
pub fn layer_norm(x: &GpuTensor, gamma: &GpuTensor, beta: &GpuTensor, eps: f32, reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let d = *x.shape().last().ok_or(NnError::DimOutOfRange { dim: 0, ndim: 0 })?;
    if gamma.numel() != d || beta.numel() != d {
        return Err(mismatch(format!("gamma/beta [{d}]"), format!("[{}] / [{}]", gamma.numel(), beta.numel())));
    }
    let y = GpuTensor::zeros(x.shape(), reg)?;
    reg.check(unsafe { sys::agpu_layer_norm(reg.raw(), x.data(), gamma.data(), beta.data(), y.data_mut(), x.rows() as i32, d as i32, eps) })?;
    Ok(y)
}

/// ops::layer_norm_residual_dual (nn/ops/norm.rs:248-400): (a + b, LayerNorm(a + b)).
pub fn layer_norm_residual_dual(a: &GpuTensor, b: &GpuTensor, gamma: &GpuTensor, beta: &GpuTensor, eps: f32,
                                reg: &Arc<KernelRegistry>) -> Result<(GpuTensor, GpuTensor)> {
    if a.shape() != b.shape() {
        return Err(mismatch(format!("{:?}", a.shape()), format!("{:?}", b.shape())));
    }
    let d = *a.shape().last().ok_or(NnError::DimOutOfRange { dim: 0, ndim: 0 })?;
    let sum = GpuTensor::zeros(a.shape(), reg)?;
    let norm = GpuTensor::zeros(a.shape(), reg)?;
    reg.check(unsafe {
        sys::agpu_add_layer_norm_dual(reg.raw(), a.data(), b.data(), gamma.data(), beta.data(), sum.data_mut(), norm.data_mut(),
                                      a.rows() as i32, d as i32, eps)
    })?;
    Ok((sum, norm))
}

/// ops::gelu (nn/ops/activation.rs:14-16, 79-108): the quick form; `gelu_tanh` is the canonical tanh form.
pub fn gelu(x: &GpuTensor, reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let y = GpuTensor::zeros(x.shape(), reg)?;
    reg.check(unsafe { sys::agpu_gelu(reg.raw(), x.data(), y.data_mut(), x.numel(), sys::AGPU_GELU_QUICK) })?;
    Ok(y)
}

pub fn gelu_tanh(x: &GpuTensor, reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let y = GpuTensor::zeros(x.shape(), reg)?;
    reg.check(unsafe { sys::agpu_gelu(reg.raw(), x.data(), y.data_mut(), x.numel(), sys::AGPU_GELU_TANH) })?;
    Ok(y)
}

/// ops::elementwise_add (nn/ops/reshape.rs:161-186): a += b.
pub fn elementwise_add(a: &mut GpuTensor, b: &GpuTensor, reg: &Arc<KernelRegistry>) -> Result<()> {
    if a.numel() != b.numel() {
        return Err(mismatch(format!("{} elements", a.numel()), format!("{} elements", b.numel())));
    }
    reg.check(unsafe { sys::agpu_add_inplace(reg.raw(), a.data_mut(), b.data(), a.numel()) })
}

/// ops::bias_add (nn/ops/reshape.rs:112-136).
pub fn bias_add(data: &mut GpuTensor, bias: &GpuTensor, reg: &Arc<KernelRegistry>) -> Result<()> {
    let n = *data.shape().last().ok_or(NnError::DimOutOfRange { dim: 0, ndim: 0 })?;
    if bias.numel() != n {
        return Err(mismatch(format!("bias [{n}]"), format!("[{}]", bias.numel())));
    }
    reg.check(unsafe { sys::agpu_bias_add(reg.raw(), data.data_mut(), bias.data(), data.rows() as i32, n as i32) })
}

/// Row softmax (CPU twin cpu_softmax_f64, nn/cpu_ref.rs:111-125).
pub fn softmax(x: &GpuTensor, reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let cols = *x.shape().last().ok_or(NnError::DimOutOfRange { dim: 0, ndim: 0 })?;
    let y = GpuTensor::zeros(x.shape(), reg)?;
    reg.check(unsafe { sys::agpu_softmax_rows(reg.raw(), x.data(), y.data_mut(), x.rows() as i32, cols as i32) })?;
    Ok(y)
}

/// ops::split_qkv (nn/ops/attention.rs:105-142): [seq, 3d] -> Q, K, V [H, seq, d_head].
pub fn split_qkv(qkv: &GpuTensor, seq_len: usize, n_heads: usize, d_head: usize, reg: &Arc<KernelRegistry>)
                 -> Result<(GpuTensor, GpuTensor, GpuTensor)> {
    if qkv.numel() != seq_len * 3 * n_heads * d_head {
        return Err(mismatch(format!("[{seq_len}, {}]", 3 * n_heads * d_head), format!("{:?}", qkv.shape())));
    }
    let shape = [n_heads, seq_len, d_head];
    let (q, k, v) = (GpuTensor::zeros(&shape, reg)?, GpuTensor::zeros(&shape, reg)?, GpuTensor::zeros(&shape, reg)?);
    reg.check(unsafe {
        sys::agpu_split_qkv(reg.raw(), qkv.data(), q.data_mut(), k.data_mut(), v.data_mut(), seq_len as i32, n_heads as i32, d_head as i32)
    })?;
    Ok((q, k, v))
}

/// ops::concat_heads (nn/ops/attention.rs:515-549): [H, seq, d_head] -> [seq, H * d_head].
pub fn concat_heads(x: &GpuTensor, seq_len: usize, n_heads: usize, d_head: usize, reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let y = GpuTensor::zeros(&[seq_len, n_heads * d_head], reg)?;
    reg.check(unsafe { sys::agpu_concat_heads(reg.raw(), x.data(), y.data_mut(), seq_len as i32, n_heads as i32, d_head as i32) })?;
    Ok(y)
}

/// ops::multi_head_flash_attention (nn/ops/attention.rs:151-202): causal attention of every head in one launch.
pub fn multi_head_flash_attention(q: &GpuTensor, k: &GpuTensor, v: &GpuTensor, seq_len: usize, n_heads: usize, d_head: usize,
                                  reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let o = GpuTensor::zeros(&[n_heads, seq_len, d_head], reg)?;
    reg.check(unsafe {
        sys::agpu_attention(reg.raw(), q.data(), k.data(), v.data(), o.data_mut(), n_heads as i32, seq_len as i32, seq_len as i32, 0,
                            seq_len as i32, d_head as i32, 1)
    })?;
    Ok(o)
}

/// ops::scaled_dot_product_attention_kv (nn/ops/attention.rs:557-606): q_len new rows at positions q_offset.. against
/// kv_len cached keys whose heads are kv_stride rows apart.
pub fn scaled_dot_product_attention_kv(q: &GpuTensor, k: &GpuTensor, v: &GpuTensor, n_heads: usize, q_len: usize, kv_len: usize,
                                       q_offset: usize, kv_stride: usize, d_head: usize, reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let o = GpuTensor::zeros(&[n_heads, q_len, d_head], reg)?;
    reg.check(unsafe {
        sys::agpu_attention(reg.raw(), q.data(), k.data(), v.data(), o.data_mut(), n_heads as i32, q_len as i32, kv_len as i32,
                            q_offset as i32, kv_stride as i32, d_head as i32, 1)
    })?;
    Ok(o)
}

/// ops::matmul (nn/ops/gemm.rs:20-212): C[M, N] = A[M, K] B[K, N] in fp32.
pub fn matmul(a: &GpuTensor, b: &GpuTensor, reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let (m, k) = (a.dim(0)?, a.dim(1)?);
    let (k2, n) = (b.dim(0)?, b.dim(1)?);
    if k != k2 {
        return Err(mismatch(format!("B [{k}, N]"), format!("[{k2}, {n}]")));
    }
    let c = GpuTensor::zeros(&[m, n], reg)?;
    reg.check(unsafe { sys::agpu_gemm_f32(reg.raw(), a.data(), b.data(), c.data_mut(), m as i32, n as i32, k as i32) })?;
    Ok(c)
}

/// quantize_weight_int4 (nn/ops/quantize.rs:102-153) on the host: weight_t [K, N] -> (packed [K/8, N], scales).
pub fn quantize_weight_int4(weight_t: &[f32], k: usize, n: usize, group_size: usize) -> Result<(Vec<u32>, Vec<f32>)> {
    if weight_t.len() != k * n || k % 8 != 0 || group_size == 0 {
        return Err(mismatch(format!("[{k}, {n}] with K % 8 == 0"), format!("{} elements", weight_t.len())));
    }
    let groups = (k + group_size - 1) / group_size;
    let mut packed = vec![0u32; k / 8 * n];
    let mut scales = vec![0f32; groups * n];
    let rc = unsafe {
        sys::agpu_int4_quantize_host(weight_t.as_ptr(), packed.as_mut_ptr(), scales.as_mut_ptr(), k as i32, n as i32, group_size as i32,
                                     sys::AGPU_QUANT_RUST)
    };
    if rc != sys::AGPU_OK {
        return Err(NnError::from_code(rc, "int4_quantize_host".to_string()));
    }
    Ok((packed, scales))
}

/// unpack_int4 (nn/ops/quantize.rs:158-162).
pub fn unpack_int4(packed: u32, index: usize) -> i8 {
    (((packed >> (index * 4)) & 0xF) as i8) - 8
}

/// argmax (nn/models/gpt2.rs:991-997) over the rows of a device tensor.
pub fn argmax_rows(x: &GpuTensor, last_index: bool, reg: &Arc<KernelRegistry>) -> Result<Vec<u32>> {
    let cols = *x.shape().last().ok_or(NnError::DimOutOfRange { dim: 0, ndim: 0 })?;
    let rows = x.rows();
    let idx = GpuTensor::zeros(&[rows], reg)?;
    reg.check(unsafe { sys::agpu_argmax_rows(reg.raw(), x.data(), idx.data_mut() as *mut u32, rows as i32, cols as i32, last_index as i32) })?;
    let mut out = vec![0u32; rows];
    reg.check(unsafe { sys::agpu_memcpy_d2h(reg.raw(), out.as_mut_ptr() as *mut std::ffi::c_void, idx.data() as *const std::ffi::c_void, rows * 4) })?;
    Ok(out)
}
