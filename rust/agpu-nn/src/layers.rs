//! nn::layers: `Module`, `Int4Linear`, `LayerNorm`, `Embedding` (nn/layers/{mod,int4_linear,norm,embedding}.rs).
use std::ffi::c_void;
use std::sync::Arc;

use agpu_sys as sys;

use crate::error::{NnError, Result};
use crate::registry::KernelRegistry;
use crate::tensor::GpuTensor;

/// trait Module (nn/layers/mod.rs:36-39).
pub trait Module {
    fn forward(&self, x: &GpuTensor) -> Result<GpuTensor>;
}

fn upload_u32(data: &[u32], reg: &Arc<KernelRegistry>) -> Result<GpuTensor> {
    let t = GpuTensor::zeros(&[data.len()], reg)?;
    reg.check(unsafe { sys::agpu_memcpy_h2d(reg.raw(), t.data_mut() as *mut c_void, data.as_ptr() as *const c_void, data.len() * 4) })?;
    Ok(t)
}

/// Int4Linear (nn/layers/int4_linear.rs:18-147): weights stay int4 in device memory, activations fp32.
pub struct Int4Linear {
    packed: GpuTensor, // [K/8, N] u32 words held in an f32-typed buffer of the same size
    scales: GpuTensor, // [ceil(K/group), N]
    bias: Option<GpuTensor>,
    in_features: usize,
    out_features: usize,
    group_size: usize,
    registry: Arc<KernelRegistry>,
}

impl Int4Linear {
    /// Int4Linear::new (int4_linear.rs:40-68).
    pub fn new(packed: &[u32], scales: &[f32], bias: Option<&[f32]>, in_features: usize, out_features: usize, group_size: usize,
               registry: &Arc<KernelRegistry>) -> Result<Int4Linear> {
        let groups = (in_features + group_size - 1) / group_size;
        if in_features % 8 != 0 || packed.len() != in_features / 8 * out_features || scales.len() != groups * out_features {
            return Err(NnError::ShapeMismatch {
                expected: format!("packed [{}, {out_features}], scales [{groups}, {out_features}]", in_features / 8),
                actual: format!("{} words, {} scales", packed.len(), scales.len()),
            });
        }
        if let Some(b) = bias {
            if b.len() != out_features {
                return Err(NnError::ShapeMismatch { expected: format!("bias [{out_features}]"), actual: format!("[{}]", b.len()) });
            }
        }
        Ok(Int4Linear {
            packed: upload_u32(packed, registry)?,
            scales: GpuTensor::from_host(scales, &[groups, out_features], registry)?,
            bias: match bias {
                Some(b) => Some(GpuTensor::from_host(b, &[out_features], registry)?),
                None => None,
            },
            in_features,
            out_features,
            group_size,
            registry: Arc::clone(registry),
        })
    }

    /// memory_bytes (int4_linear.rs:136-146).
    pub fn memory_bytes(&self) -> usize {
        self.packed.numel() * 4 + self.scales.numel() * 4 + self.bias.as_ref().map(|b| b.numel() * 4).unwrap_or(0)
    }
    pub fn in_features(&self) -> usize {
        self.in_features
    }
    pub fn out_features(&self) -> usize {
        self.out_features
    }
}

impl Module for Int4Linear {
    /// Int4Linear::forward (int4_linear.rs:71-133): [*, K] -> [*, N], bias added by the same launch.
    fn forward(&self, x: &GpuTensor) -> Result<GpuTensor> {
        let k = *x.shape().last().ok_or(NnError::DimOutOfRange { dim: 0, ndim: 0 })?;
        if k != self.in_features {
            return Err(NnError::ShapeMismatch { expected: format!("[*, {}]", self.in_features), actual: format!("{:?}", x.shape()) });
        }
        let mut shape = x.shape().to_vec();
        *shape.last_mut().unwrap() = self.out_features;
        let y = GpuTensor::zeros(&shape, &self.registry)?;
        let reg = &self.registry;
        reg.check(unsafe {
            sys::agpu_int4_linear(reg.raw(), x.data(), self.packed.data() as *const u32, self.scales.data(),
                                  self.bias.as_ref().map(|b| b.data()).unwrap_or(std::ptr::null()), std::ptr::null(), y.data_mut(),
                                  x.rows() as i32, self.out_features as i32, self.in_features as i32, self.group_size as i32,
                                  sys::AGPU_EPI_NONE)
        })?;
        Ok(y)
    }
}

/// LayerNorm (nn/layers/norm.rs:15-55).
pub struct LayerNorm {
    gamma: GpuTensor,
    beta: GpuTensor,
    eps: f32,
    registry: Arc<KernelRegistry>,
}

impl LayerNorm {
    pub fn new(gamma: &[f32], beta: &[f32], eps: f32, registry: &Arc<KernelRegistry>) -> Result<LayerNorm> {
        if gamma.len() != beta.len() {
            return Err(NnError::ShapeMismatch { expected: format!("beta [{}]", gamma.len()), actual: format!("[{}]", beta.len()) });
        }
        Ok(LayerNorm {
            gamma: GpuTensor::from_host(gamma, &[gamma.len()], registry)?,
            beta: GpuTensor::from_host(beta, &[beta.len()], registry)?,
            eps,
            registry: Arc::clone(registry),
        })
    }
}

impl Module for LayerNorm {
    fn forward(&self, x: &GpuTensor) -> Result<GpuTensor> {
        crate::ops::layer_norm(x, &self.gamma, &self.beta, self.eps, &self.registry)
    }
}

/// Embedding (nn/layers/embedding.rs:15-93): wte[token] + wpe[position + offset].
pub struct Embedding {
    wte: GpuTensor,
    wpe: GpuTensor,
    d_model: usize,
    vocab_size: usize,
    n_positions: usize,
    registry: Arc<KernelRegistry>,
}

impl Embedding {
    pub fn new(wte: &[f32], wpe: &[f32], vocab_size: usize, n_positions: usize, d_model: usize, registry: &Arc<KernelRegistry>)
               -> Result<Embedding> {
        Ok(Embedding {
            wte: GpuTensor::from_host(wte, &[vocab_size, d_model], registry)?,
            wpe: GpuTensor::from_host(wpe, &[n_positions, d_model], registry)?,
            d_model,
            vocab_size,
            n_positions,
            registry: Arc::clone(registry),
        })
    }

    /// forward_tokens (embedding.rs:46-57).
    pub fn forward_tokens(&self, tokens: &[u32]) -> Result<GpuTensor> {
        self.forward_tokens_with_offset(tokens, 0)
    }

    /// forward_tokens_with_offset (embedding.rs:59-93); ids and positions are checked here, where the host knows them.
    pub fn forward_tokens_with_offset(&self, tokens: &[u32], pos_offset: usize) -> Result<GpuTensor> {
        if let Some(&bad) = tokens.iter().find(|&&t| t as usize >= self.vocab_size) {
            return Err(NnError::Library { code: sys::AGPU_ERR_DIM_OUT_OF_RANGE, message: format!("token id {bad} outside the vocabulary of {}", self.vocab_size) });
        }
        if pos_offset + tokens.len() > self.n_positions {
            return Err(NnError::Library { code: sys::AGPU_ERR_DIM_OUT_OF_RANGE, message: format!("{} positions exceed n_positions {}", pos_offset + tokens.len(), self.n_positions) });
        }
        let reg = &self.registry;
        let ids = upload_u32(tokens, reg)?;
        let out = GpuTensor::zeros(&[tokens.len(), self.d_model], reg)?;
        reg.check(unsafe {
            sys::agpu_embedding(reg.raw(), ids.data() as *const u32, self.wte.data(), self.wpe.data(), out.data_mut(), tokens.len() as i32,
                                self.d_model as i32, pos_offset as i32)
        })?;
        Ok(out)
    }
}
