//! MI355X implementation of rustllm-core's transformer model plugin: the same traits and the same
//! plugin id as `plugins/model-transformer`, over the C ABI of `include/coeus.h`
//! (libcoeus_mi355x.so).  Source only: the image this library is built in has no Rust toolchain,
//! so this crate has not been compiled there.
pub mod tokenizer;

use rustllm_core::core::model::{ForwardModel, Model, ModelBuilder, Transformer250MConfig};
use rustllm_core::core::plugin::{ModelBuilderPlugin, Plugin, PluginCapabilities};
use rustllm_core::core::traits::{Identity, Versioned};
use rustllm_core::foundation::{error::{invalid_input, internal_error, ConfigError, Error, Result},
                               types::Version};
use std::ffi::CStr;
use std::os::raw::{c_char, c_int};

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct CoeusConfig {          // include/coeus.h: coeus_config
    hidden_dim: u64, num_layers: u64, num_heads: u64, intermediate_dim: u64,
    vocab_size: u64, max_seq_len: u64,
    dropout: f32, attention_dropout: f32, layer_norm_eps: f32, use_bias: u8,
    activation: u32, norm: u32, norm_scope: u32, weight_dtype: u32, kv_dtype: u32,
    head_dim: u64, max_batch: u64,
}
// Layout of coeus_config as the C compiler lays out include/coeus.h on x86-64; a change of the
// struct above that moves a field fails to compile here (tests/test_abi_layout.py checks these
// figures and the field list against sizeof / offsetof of the header).
pub const COEUS_CONFIG_SIZE: usize = 104;
pub const COEUS_CONFIG_OFFSET_USE_BIAS: usize = 60;
pub const COEUS_CONFIG_OFFSET_ACTIVATION: usize = 64;
pub const COEUS_CONFIG_OFFSET_HEAD_DIM: usize = 88;
const _: () = assert!(std::mem::size_of::<CoeusConfig>() == COEUS_CONFIG_SIZE);
const _: () = assert!(std::mem::align_of::<CoeusConfig>() == 8);
#[repr(C)] pub struct CoeusModel { _private: [u8; 0] }

#[link(name = "coeus_mi355x")]
extern "C" {
    fn coeus_last_error() -> *const c_char;
    fn coeus_config_validate(cfg: *const CoeusConfig) -> c_int;
    fn coeus_config_num_parameters(cfg: *const CoeusConfig) -> u64;
    fn coeus_init_default_parameters(params: *mut f32, n: u64, hidden_dim: u64) -> c_int;
    fn coeus_model_create(cfg: *const CoeusConfig, params: *const f32, n: u64,
                          out: *mut *mut CoeusModel) -> c_int;
    fn coeus_model_forward(m: *mut CoeusModel, ids: *const u64, n: u64, logits: *mut f32) -> c_int;
    fn coeus_model_destroy(m: *mut CoeusModel);
}

fn check(rc: c_int) -> Result<()> {
    if rc == 0 { return Ok(()); }
    let msg = unsafe { CStr::from_ptr(coeus_last_error()) }.to_string_lossy().into_owned();
    Err(match rc {
        1 => invalid_input(msg),                                   // COEUS_INVALID_INPUT
        2 => Error::Config(ConfigError::Invalid {                  // COEUS_INVALID_CONFIG
                 key: "config".into(), value: String::new(), error: msg }),
        _ => internal_error(msg),                                  // device / out of memory
    })
}

fn to_c(c: &Transformer250MConfig) -> CoeusConfig {
    CoeusConfig { hidden_dim: c.hidden_dim as u64, num_layers: c.num_layers as u64,
                  num_heads: c.num_heads as u64, intermediate_dim: c.intermediate_dim as u64,
                  vocab_size: c.vocab_size as u64, max_seq_len: c.max_seq_len as u64,
                  dropout: c.dropout, attention_dropout: c.attention_dropout,
                  layer_norm_eps: c.layer_norm_eps, use_bias: c.use_bias as u8,
                  ..Default::default() }          // extension fields 0 = the reference's behaviour
}

#[derive(Debug, Default)] pub struct TransformerModelPlugin;
impl Identity for TransformerModelPlugin { fn id(&self) -> &str { "transformer_model" } }
impl Versioned for TransformerModelPlugin { fn version(&self) -> Version { Version::new(0, 1, 0) } }
impl Plugin for TransformerModelPlugin {
    fn capabilities(&self) -> PluginCapabilities {
        PluginCapabilities::standard().with_feature("model_building")
            .with_feature("transformer").with_feature("250M_params")
    }
}
impl ModelBuilderPlugin for TransformerModelPlugin {
    type Builder = TransformerModelBuilder;
    fn create_builder(&self) -> Result<Self::Builder> { Ok(TransformerModelBuilder) }
}

#[derive(Debug, Default)] pub struct TransformerModelBuilder;
impl ModelBuilder for TransformerModelBuilder {
    type Model = TransformerModel;
    type Config = Transformer250MConfig;
    fn build(&self, config: Self::Config) -> Result<Self::Model> {
        let c = to_c(&config);
        check(unsafe { coeus_config_validate(&c) })?;
        let n = unsafe { coeus_config_num_parameters(&c) } as usize;
        let mut params = vec![0.0f32; n];
        check(unsafe { coeus_init_default_parameters(params.as_mut_ptr(), n as u64, c.hidden_dim) })?;
        let mut h = std::ptr::null_mut();
        check(unsafe { coeus_model_create(&c, params.as_ptr(), n as u64, &mut h) })?;
        Ok(TransformerModel { config, handle: h, n_params: n })   // weights now live in HBM
    }
}

#[derive(Debug)]
pub struct TransformerModel { config: Transformer250MConfig, handle: *mut CoeusModel, n_params: usize }
unsafe impl Send for TransformerModel {}   // the library serialises calls on one model
unsafe impl Sync for TransformerModel {}
impl Drop for TransformerModel { fn drop(&mut self) { unsafe { coeus_model_destroy(self.handle) } } }
impl Model for TransformerModel {
    type Config = Transformer250MConfig;
    fn config(&self) -> &Self::Config { &self.config }
    fn name(&self) -> &str { "TransformerModel" }
}
impl ForwardModel for TransformerModel {
    type Input = Vec<usize>;
    type Output = Vec<f32>;
    fn forward(&self, input: Self::Input) -> Result<Self::Output> {
        let ids: Vec<u64> = input.iter().map(|&t| t as u64).collect();
        let mut logits = vec![0.0f32; self.config.vocab_size];
        check(unsafe { coeus_model_forward(self.handle, ids.as_ptr(), ids.len() as u64,
                                           logits.as_mut_ptr()) })?;
        Ok(logits)
    }
    fn num_parameters(&self) -> usize { self.n_params }
}

// ---- weights from a `.rustllm` file (lib.rs:1008-1121 over the C ABI's reader) ----------------
extern "C" {
    fn coeus_rustllm_read_header(path: *const c_char, cfg: *mut CoeusConfig, n: *mut u64) -> c_int;
    fn coeus_rustllm_read_parameters(path: *const c_char, params: *mut f32, n: u64) -> c_int;
    fn coeus_rustllm_write(path: *const c_char, cfg: *const CoeusConfig, params: *const f32, n: u64) -> c_int;
}

impl TransformerModelBuilder {
    /// `build` with caller-supplied parameters in the layout of lib.rs:677-740 (what `read_from`
    /// produces); the buffer may be dropped after the call, the weights live in HBM.
    pub fn build_with_parameters(&self, config: Transformer250MConfig, params: &[f32]) -> Result<TransformerModel> {
        let c = to_c(&config);
        check(unsafe { coeus_config_validate(&c) })?;
        let mut h = std::ptr::null_mut();
        check(unsafe { coeus_model_create(&c, params.as_ptr(), params.len() as u64, &mut h) })?;
        Ok(TransformerModel { config, handle: h, n_params: params.len() })
    }

    /// Reads header, checksummed parameters and metadata of a `.rustllm` file and builds the model.
    pub fn load(&self, path: &std::path::Path) -> Result<TransformerModel> {
        let p = std::ffi::CString::new(path.to_string_lossy().as_bytes()).map_err(|e| invalid_input(e.to_string()))?;
        let mut c = CoeusConfig::default();
        let mut n = 0u64;
        check(unsafe { coeus_rustllm_read_header(p.as_ptr(), &mut c, &mut n) })?;
        let mut params = vec![0.0f32; n as usize];
        check(unsafe { coeus_rustllm_read_parameters(p.as_ptr(), params.as_mut_ptr(), n) })?;
        let config = Transformer250MConfig {
            hidden_dim: c.hidden_dim as usize, num_layers: c.num_layers as usize,
            num_heads: c.num_heads as usize, intermediate_dim: c.intermediate_dim as usize,
            vocab_size: c.vocab_size as usize, max_seq_len: c.max_seq_len as usize,
            layer_norm_eps: c.layer_norm_eps, use_bias: c.use_bias != 0,
            ..Transformer250MConfig::default()
        };
        // The model is created from the config the reader returned, not from `to_c(&config)`:
        // Transformer250MConfig has no field for the extension keys (activation, norm, norm_scope,
        // head_dim, weight/kv dtype), and rebuilding the C struct from it would zero them, so a
        // file written from a gated / RMS-norm model would load as a different parameter layout.
        check(unsafe { coeus_config_validate(&c) })?;
        let mut h = std::ptr::null_mut();
        check(unsafe { coeus_model_create(&c, params.as_ptr(), params.len() as u64, &mut h) })?;
        Ok(TransformerModel { config, handle: h, n_params: params.len() })
    }
}

/// Writes `params` (the vector a model was built from) as a `.rustllm` file (lib.rs:931-1006).
pub fn write_rustllm(path: &std::path::Path, config: &Transformer250MConfig, params: &[f32]) -> Result<()> {
    let p = std::ffi::CString::new(path.to_string_lossy().as_bytes()).map_err(|e| invalid_input(e.to_string()))?;
    let c = to_c(config);
    check(unsafe { coeus_rustllm_write(p.as_ptr(), &c, params.as_ptr(), params.len() as u64) })
}
