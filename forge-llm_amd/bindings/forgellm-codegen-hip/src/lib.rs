//! Forge HIP code generation: AMD MI355X (gfx950) inference through `libforge_hip`.
//!
//! Like the Metal generator this crate writes a complete Cargo project, but the project holds no kernels: its
//! `src/model.rs` binds the C ABI of `libforge_hip.so` (`include/forge_hip.h`) and exposes `HipModel` with the surface of
//! `MetalModel` (`new`, `forward`, `forward_prefill_batch`, `reset`), and its `src/main.rs` is the generated CLI
//! (same flags and defaults as the CPU and Metal projects).
//!
//! Wiring in `forgellm-cli` (`cmd_compile`, the `match target.as_str()` next to `"metal"`):
//!
//! ```ignore
//! "hip" => forgellm_codegen_hip::generate_hip_project(&graph, &output_dir, &model_name)
//!     .map_err(|e| anyhow::anyhow!("HIP codegen failed: {e}"))?,
//! ```

use std::fs;
use std::path::Path;

use forgellm_frontend::ir::*;

/// Errors during HIP code generation.
#[derive(Debug, thiserror::Error)]
pub enum HipCodegenError {
    /// The computation graph has no attached [`ModelConfig`].
    #[error("graph has no model config")]
    MissingConfig,

    /// The model is outside what `libforge_hip` runs.
    #[error("unsupported model for the HIP backend: {0}")]
    Unsupported(String),

    /// An I/O error during file creation.
    #[error("I/O error: {0}")]
    Io(#[from] std::io::Error),
}

/// GGML type ids `libforge_hip` takes for `wdtype` / `lm_head_dtype`.
const FORGE_HIP_Q4_0: u32 = 2;
const FORGE_HIP_Q8_0: u32 = 8;
/// `config.flags` bit: the blob carries Qwen2's QKV bias vectors.
const FORGE_HIP_FLAG_QKV_BIAS: u32 = 2;

/// Generate a complete HIP Cargo project from a computation graph.
///
/// Creates `Cargo.toml`, `build.rs` (links `forge_hip`; the directory comes from `FORGE_HIP_LIB_DIR`), `src/model.rs`
/// (the binding and `HipModel`) and `src/main.rs` (the CLI).
pub fn generate_hip_project(graph: &Graph, output_dir: &Path, model_name: &str) -> Result<(), HipCodegenError> {
    let config = graph.config.as_ref().ok_or(HipCodegenError::MissingConfig)?;
    let src_dir = output_dir.join("src");
    fs::create_dir_all(&src_dir)?;
    fs::write(output_dir.join("Cargo.toml"), generate_cargo_toml(model_name))?;
    fs::write(output_dir.join("build.rs"), BUILD_RS)?;
    fs::write(src_dir.join("model.rs"), generate_model_rs(config)?)?;
    fs::write(src_dir.join("main.rs"), generate_main_rs(model_name, config))?;
    Ok(())
}

fn sanitize_name(name: &str) -> String {
    let s: String = name
        .to_lowercase()
        .chars()
        .map(|c| if c.is_ascii_alphanumeric() || c == '-' { c } else { '-' })
        .collect();
    let s = s.trim_matches('-').to_string();
    if s.is_empty() { "forge-model".to_string() } else { s }
}

fn ggml_type_of(dtype: DType) -> Result<u32, HipCodegenError> {
    match dtype {
        DType::Q8_0 => Ok(FORGE_HIP_Q8_0),
        DType::Q4_0 => Ok(FORGE_HIP_Q4_0),
        other => Err(HipCodegenError::Unsupported(format!(
            "weights of type {other:?}: libforge_hip takes Q8_0 or Q4_0 projections"
        ))),
    }
}

/// `Cargo.toml` of the generated project.
pub fn generate_cargo_toml(model_name: &str) -> String {
    CARGO_TOML.replace("@NAME@", &sanitize_name(model_name))
}

/// `src/model.rs` of the generated project: constants from the [`ModelConfig`], the `extern "C"` block and `HipModel`.
pub fn generate_model_rs(config: &ModelConfig) -> Result<String, HipCodegenError> {
    let wdtype = ggml_type_of(config.dtype)?;
    let lm_head_dtype = match config.lm_head_dtype {
        Some(d) => ggml_type_of(d)?,
        None => wdtype,
    };
    if config.proj_dtypes.is_some() {
        return Err(HipCodegenError::Unsupported("per-projection dtypes (K-quant models)".to_string()));
    }
    if !matches!(config.hidden_activation, HiddenActivation::SiLU) {
        return Err(HipCodegenError::Unsupported("a GeLU feed-forward block".to_string()));
    }
    if ![64usize, 96, 128].contains(&config.head_dim) {
        return Err(HipCodegenError::Unsupported(format!("head_dim {} (64, 96 or 128)", config.head_dim)));
    }
    let flags = if config.qkv_bias { FORGE_HIP_FLAG_QKV_BIAS } else { 0 };
    Ok(MODEL_RS
        .replace("@HIDDEN@", &config.hidden_size.to_string())
        .replace("@INTER@", &config.intermediate_size.to_string())
        .replace("@LAYERS@", &config.num_layers.to_string())
        .replace("@HEADS@", &config.num_attention_heads.to_string())
        .replace("@KV_HEADS@", &config.num_kv_heads.to_string())
        .replace("@HEAD_DIM@", &config.head_dim.to_string())
        .replace("@VOCAB@", &config.vocab_size.to_string())
        .replace("@MAX_SEQ@", &config.max_seq_len.to_string())
        .replace("@RMS_EPS@", &format!("{:e}", config.rms_norm_eps))
        .replace("@ROPE_THETA@", &format!("{:e}", config.rope_theta))
        .replace("@WDTYPE@", &wdtype.to_string())
        .replace("@LM_HEAD_DTYPE@", &lm_head_dtype.to_string())
        .replace("@FLAGS@", &flags.to_string())
        .replace("@SLIDING_WINDOW@", &config.sliding_window_size.unwrap_or(0).to_string()))
}

/// `src/main.rs` of the generated project.
pub fn generate_main_rs(model_name: &str, config: &ModelConfig) -> String {
    MAIN_RS
        .replace("@MODEL_NAME@", &model_name.replace('"', "'"))
        .replace("@ARCH@", &format!("{:?}", config.architecture))
        .replace("@LAYERS@", &config.num_layers.to_string())
        .replace("@HIDDEN@", &config.hidden_size.to_string())
}

const CARGO_TOML: &str = r#"[package]
name = "@NAME@"
version = "0.1.0"
edition = "2021"

[dependencies]
tokenizers = { version = "0.21", default-features = false, features = ["onig"] }

[profile.release]
opt-level = 3
lto = true
"#;

const BUILD_RS: &str = r#"// libforge_hip.so is built from the forge-llm_amd sources (python -m forge-llm_amd.build); point FORGE_HIP_LIB_DIR at its directory.
fn main() {
    println!("cargo:rerun-if-env-changed=FORGE_HIP_LIB_DIR");
    if let Ok(dir) = std::env::var("FORGE_HIP_LIB_DIR") {
        println!("cargo:rustc-link-search=native={dir}");
        println!("cargo:rustc-link-arg=-Wl,-rpath,{dir}");
    }
    println!("cargo:rustc-link-lib=dylib=forge_hip");
}
"#;

const MODEL_RS: &str = r#"//! Binding of libforge_hip (include/forge_hip.h) and `HipModel`, the counterpart of `MetalModel`.
#![allow(dead_code)]

use std::ffi::{CStr, CString};
use std::os::raw::c_char;

pub const HIDDEN_SIZE: usize = @HIDDEN@;
pub const INTERMEDIATE_SIZE: usize = @INTER@;
pub const NUM_LAYERS: usize = @LAYERS@;
pub const NUM_HEADS: usize = @HEADS@;
pub const NUM_KV_HEADS: usize = @KV_HEADS@;
pub const HEAD_DIM: usize = @HEAD_DIM@;
pub const VOCAB_SIZE: usize = @VOCAB@;
pub const MAX_SEQ_LEN: usize = @MAX_SEQ@;
pub const RMS_NORM_EPS: f32 = @RMS_EPS@;
pub const ROPE_THETA: f32 = @ROPE_THETA@;
pub const SLIDING_WINDOW_SIZE: usize = @SLIDING_WINDOW@;  // 0 = full attention
pub const WDTYPE: u32 = @WDTYPE@;          // GGML type id of the projections: 8 = Q8_0, 2 = Q4_0
pub const LM_HEAD_DTYPE: u32 = @LM_HEAD_DTYPE@;
pub const FLAGS: u32 = @FLAGS@;            // bit 2: QKV bias (Qwen2)

#[repr(C)]
pub struct ForgeHipConfig {
    pub hidden: u32,
    pub inter: u32,
    pub layers: u32,
    pub heads: u32,
    pub kv_heads: u32,
    pub head_dim: u32,
    pub vocab: u32,
    pub max_seq: u32,
    pub rms_eps: f32,
    pub rope_theta: f32,
    pub wdtype: u32,
    pub lm_head_dtype: u32,
    pub flags: u32,
    pub sliding_window: u32,
}

#[repr(C)]
pub struct ForgeHipModel {
    _private: [u8; 0],
}

extern "C" {
    fn forge_hip_last_error() -> *const c_char;
    fn forge_hip_device_count() -> i32;
    fn forge_hip_weights_nbytes(cfg: *const ForgeHipConfig) -> u64;
    fn forge_hip_model_create(cfg: *const ForgeHipConfig, weights_bin_host: *const u8, nbytes: u64, out: *mut *mut ForgeHipModel) -> i32;
    fn forge_hip_model_create_from_gguf(path: *const c_char, max_seq: u32, flags: u32, out: *mut *mut ForgeHipModel) -> i32;
    fn forge_hip_model_destroy(m: *mut ForgeHipModel);
    fn forge_hip_forward(m: *mut ForgeHipModel, token: u32, logits_host: *mut f32) -> i32;
    fn forge_hip_forward_greedy(m: *mut ForgeHipModel, token: u32, next_token_host: *mut u32) -> i32;
    fn forge_hip_prefill_batch(m: *mut ForgeHipModel, tokens_host: *const u32, n: u64, logits_host: *mut f32) -> i32;
    fn forge_hip_reset(m: *mut ForgeHipModel) -> i32;
    fn forge_hip_model_pos(m: *const ForgeHipModel) -> i64;
    fn forge_hip_model_set_repeat_penalty(m: *mut ForgeHipModel, penalty: f32) -> i32;
    fn forge_hip_apply_repeat_penalty(logits_host: *mut f32, n: u64, recent_host: *const u32, n_recent: u64, penalty: f32) -> i32;
    fn forge_hip_sample(logits_host: *mut f32, n: u64, temperature: f32, top_k: u64, top_p: f32, rng_state: *mut u64, out: *mut u32) -> i32;
}

fn last_error() -> String {
    unsafe { CStr::from_ptr(forge_hip_last_error()) }.to_string_lossy().into_owned()
}

fn check(rc: i32) {
    if rc != 0 {
        panic!("libforge_hip: {} (code {})", last_error(), rc);
    }
}

pub fn config() -> ForgeHipConfig {
    ForgeHipConfig {
        hidden: HIDDEN_SIZE as u32,
        inter: INTERMEDIATE_SIZE as u32,
        layers: NUM_LAYERS as u32,
        heads: NUM_HEADS as u32,
        kv_heads: NUM_KV_HEADS as u32,
        head_dim: HEAD_DIM as u32,
        vocab: VOCAB_SIZE as u32,
        max_seq: MAX_SEQ_LEN as u32,
        rms_eps: RMS_NORM_EPS,
        rope_theta: ROPE_THETA,
        wdtype: WDTYPE,
        lm_head_dtype: LM_HEAD_DTYPE,
        flags: FLAGS,
        sliding_window: SLIDING_WINDOW_SIZE as u32,
    }
}

/// The model on the GPU.  Same surface as `MetalModel`; one caller thread per model.
pub struct HipModel {
    h: *mut ForgeHipModel,
}

impl HipModel {
    /// `weights` is the file `forge export-weights` writes.  Panics, like the other backends, if it does not fit the model.
    pub fn new(weights: &[u8]) -> Self {
        let cfg = config();
        let need = unsafe { forge_hip_weights_nbytes(&cfg) };
        if need != weights.len() as u64 {
            panic!("weights file is {} bytes, the compiled model needs {}", weights.len(), need);
        }
        let mut h: *mut ForgeHipModel = std::ptr::null_mut();
        check(unsafe { forge_hip_model_create(&cfg, weights.as_ptr(), weights.len() as u64, &mut h) });
        HipModel { h }
    }

    /// Straight from a GGUF file (the library does parse, load_config and export-weights itself).
    pub fn from_gguf(path: &str) -> Self {
        let c = CString::new(path).expect("path contains a NUL byte");
        let mut h: *mut ForgeHipModel = std::ptr::null_mut();
        check(unsafe { forge_hip_model_create_from_gguf(c.as_ptr(), MAX_SEQ_LEN as u32, 0, &mut h) });
        HipModel { h }
    }

    /// One decode step at the current position: logits of the next token.
    pub fn forward(&mut self, token_id: u32) -> Vec<f32> {
        let mut logits = vec![0.0f32; VOCAB_SIZE];
        check(unsafe { forge_hip_forward(self.h, token_id, logits.as_mut_ptr()) });
        logits
    }

    /// One decode step with the argmax (and the repeat penalty set with `set_repeat_penalty`) taken on the GPU: 4 bytes
    /// come back instead of the logits.
    pub fn forward_greedy(&mut self, token_id: u32) -> u32 {
        let mut next = 0u32;
        check(unsafe { forge_hip_forward_greedy(self.h, token_id, &mut next) });
        next
    }

    /// Fills the KV cache for `tokens` from the current position.
    pub fn forward_prefill_batch(&mut self, tokens: &[u32]) {
        check(unsafe { forge_hip_prefill_batch(self.h, tokens.as_ptr(), tokens.len() as u64, std::ptr::null_mut()) });
    }

    /// Batched prefill that also returns the logits of the last token (the CPU backend's `forward_prefill`).
    pub fn forward_prefill(&mut self, tokens: &[u32]) -> Vec<f32> {
        let mut logits = vec![0.0f32; VOCAB_SIZE];
        check(unsafe { forge_hip_prefill_batch(self.h, tokens.as_ptr(), tokens.len() as u64, logits.as_mut_ptr()) });
        logits
    }

    pub fn set_repeat_penalty(&mut self, penalty: f32) {
        check(unsafe { forge_hip_model_set_repeat_penalty(self.h, penalty) });
    }

    pub fn pos(&self) -> usize {
        unsafe { forge_hip_model_pos(self.h) as usize }
    }

    pub fn reset(&mut self) {
        check(unsafe { forge_hip_reset(self.h) });
    }
}

impl Drop for HipModel {
    fn drop(&mut self) {
        unsafe { forge_hip_model_destroy(self.h) }
    }
}

pub fn device_count() -> i32 {
    unsafe { forge_hip_device_count() }
}

/// `apply_repeat_penalty` of the generated CPU project, run by the library on host logits.
pub fn apply_repeat_penalty(logits: &mut [f32], recent: &[u32], penalty: f32) {
    check(unsafe { forge_hip_apply_repeat_penalty(logits.as_mut_ptr(), logits.len() as u64, recent.as_ptr(), recent.len() as u64, penalty) });
}

/// `sample` of the generated CPU project (temperature, top-k, top-p, xorshift64), run by the library on host logits.
pub fn sample(logits: &mut [f32], temperature: f32, top_k: usize, top_p: f32, rng_state: &mut u64) -> u32 {
    let mut out = 0u32;
    check(unsafe { forge_hip_sample(logits.as_mut_ptr(), logits.len() as u64, temperature, top_k as u64, top_p, rng_state, &mut out) });
    out
}
"#;

const MAIN_RS: &str = r#"//! @MODEL_NAME@ on AMD MI355X through libforge_hip.  Generated by forgellm-codegen-hip.
//!
//! Same command line as the binaries of the other ForgeLLM backends (flags, defaults, what goes to stdout and what to
//! stderr); the first argument may also be a GGUF file.
mod model;

use std::io::Write;
use std::time::Instant;

use model::{apply_repeat_penalty, sample, HipModel};

/// Everything the command line can say.  Defaults are those of the CPU backend's binary.
struct Options {
    weights: String,
    tokenizer: String,
    prompt: String,
    temperature: f32,
    top_k: usize,
    top_p: f32,
    max_tokens: usize,
    repeat_penalty: f32,
    seed: u64,
    quiet: bool,
}

const USAGE_FLAGS: &str = "[prompt] [--temp T] [--top-k K] [--top-p P] [--max-tokens N] [--repeat-penalty R] [--seed S] [--quiet]";

impl Options {
    /// One pass over the arguments after the two paths: `--flag value` pairs fill their field (a value that does not parse
    /// leaves the default), `--quiet` / `-q` is a switch, any other dash argument is skipped, the rest is the prompt.
    fn from_args(args: &[String]) -> Options {
        let mut o = Options {
            weights: args[1].clone(),
            tokenizer: args[2].clone(),
            prompt: String::new(),
            temperature: 0.0,
            top_k: 0,
            top_p: 0.9,
            max_tokens: 128,
            repeat_penalty: 1.1,
            seed: 0xdeadbeef12345678,
            quiet: false,
        };
        let mut words: Vec<&str> = Vec::new();
        let mut rest = args[3..].iter();
        while let Some(arg) = rest.next() {
            match arg.as_str() {
                "--quiet" | "-q" => o.quiet = true,
                "--temp" => set(&mut o.temperature, rest.next()),
                "--top-k" => set(&mut o.top_k, rest.next()),
                "--top-p" => set(&mut o.top_p, rest.next()),
                "--max-tokens" => set(&mut o.max_tokens, rest.next()),
                "--repeat-penalty" => set(&mut o.repeat_penalty, rest.next()),
                "--seed" => set(&mut o.seed, rest.next()),
                other if other.starts_with('-') => {}
                word => words.push(word),
            }
        }
        o.prompt = if words.is_empty() { "Hello".to_string() } else { words.join(" ") };
        o
    }
}

fn set<T: std::str::FromStr>(field: &mut T, value: Option<&String>) {
    if let Some(v) = value.and_then(|v| v.parse::<T>().ok()) {
        *field = v;
    }
}

fn main() {
    let args: Vec<String> = std::env::args().collect();
    if args.iter().any(|a| a == "--version" || a == "-V") {
        println!("@MODEL_NAME@ (ForgeLLM, HIP backend)");
        return;
    }
    if args.len() < 3 {
        eprintln!("Usage: {} <weights.bin | model.gguf> <tokenizer.json> {}", args[0], USAGE_FLAGS);
        eprintln!("AOT-compiled @ARCH@ | @LAYERS@ layers | hidden=@HIDDEN@ | HIP (gfx950)");
        std::process::exit(1);
    }
    let opt = Options::from_args(&args);
    if model::device_count() < 1 {
        eprintln!("no AMD GPU visible to HIP");
        std::process::exit(1);
    }
    let tokenizer = tokenizers::Tokenizer::from_file(&opt.tokenizer).expect("failed to load tokenizer");
    let mut gpu = if opt.weights.ends_with(".gguf") {
        HipModel::from_gguf(&opt.weights)
    } else {
        HipModel::new(&std::fs::read(&opt.weights).expect("failed to read weights"))
    };

    let prompt_ids: Vec<u32> = tokenizer.encode(opt.prompt.as_str(), false).expect("encode failed").get_ids().to_vec();
    eprintln!("Prompt: {} tokens | temp={} top_k={} max_tokens={}", prompt_ids.len(), opt.temperature, opt.top_k, opt.max_tokens);

    // prompt in one batched pass; the first token is sampled from its logits without a penalty
    let mut rng = opt.seed;
    let started = Instant::now();
    let mut first_logits = gpu.forward_prefill(&prompt_ids);
    let first = sample(&mut first_logits, opt.temperature, opt.top_k, opt.top_p, &mut rng);
    eprintln!("Prefill: {:.1} tok/s", prompt_ids.len() as f64 / started.elapsed().as_secs_f64());

    if !opt.quiet {
        print!("{}", opt.prompt);
    }
    let started = Instant::now();
    let produced = generate(&mut gpu, &tokenizer, &opt, prompt_ids, first, &mut rng);
    if !opt.quiet {
        println!();
    }
    let secs = started.elapsed().as_secs_f64();
    eprintln!("Generate: {} tokens in {:.2}s ({:.1} tok/s)", produced, secs, produced as f64 / secs);
}

/// Feeds `token`, then whatever is chosen next, until an end-of-sequence id or `max_tokens`; returns how many were fed.
/// With temperature <= 0 the choice stays on the GPU: the library counts every token it has been fed (the prompt's too) and
/// takes the argmax of the penalised logits itself, so 4 bytes per token come back.  Otherwise the logits come back and the
/// penalty over all tokens so far and the sampler run here.
fn generate(gpu: &mut HipModel, tokenizer: &tokenizers::Tokenizer, opt: &Options, prompt_ids: Vec<u32>, first: u32, rng: &mut u64) -> usize {
    let stop: Vec<u32> = ["</s>", "<|endoftext|>", "<|im_end|>", "<|eot_id|>"].iter().filter_map(|t| tokenizer.token_to_id(t)).collect();
    let on_gpu = opt.temperature <= 0.0;
    if on_gpu {
        gpu.set_repeat_penalty(opt.repeat_penalty);
    }
    let mut seen = prompt_ids;
    let mut token = first;
    let mut fed = 0usize;
    while fed < opt.max_tokens && !stop.contains(&token) {
        if !opt.quiet {
            print!("{}", tokenizer.decode(&[token], true).unwrap_or_default());
            std::io::stdout().flush().ok();
        }
        seen.push(token);
        token = if on_gpu {
            gpu.forward_greedy(token)
        } else {
            let mut logits = gpu.forward(token);
            apply_repeat_penalty(&mut logits, &seen, opt.repeat_penalty);
            sample(&mut logits, opt.temperature, opt.top_k, opt.top_p, rng)
        };
        fed += 1;
    }
    fed
}
"#;

#[cfg(test)]
mod tests {
    use super::*;

    fn test_config() -> ModelConfig {
        ModelConfig {
            architecture: Architecture::Llama,
            hidden_size: 2048,
            intermediate_size: 8192,
            num_layers: 16,
            num_attention_heads: 32,
            num_kv_heads: 8,
            head_dim: 64,
            vocab_size: 128256,
            max_seq_len: 4096,
            rms_norm_eps: 1e-5,
            rope_theta: 500000.0,
            dtype: DType::Q8_0,
            lm_head_dtype: None,
            proj_dtypes: None,
            sliding_window_size: None,
            qkv_bias: false,
            hidden_activation: HiddenActivation::SiLU,
        }
    }

    #[test]
    fn model_rs_carries_the_constants_and_the_binding() {
        let code = generate_model_rs(&test_config()).unwrap();
        assert!(code.contains("pub const HIDDEN_SIZE: usize = 2048;"));
        assert!(code.contains("pub const NUM_KV_HEADS: usize = 8;"));
        assert!(code.contains("pub const WDTYPE: u32 = 8;"));
        assert!(code.contains("pub const LM_HEAD_DTYPE: u32 = 8;"));
        assert!(code.contains("pub const SLIDING_WINDOW_SIZE: usize = 0;"));
        assert!(code.contains("fn forge_hip_model_create("));
        assert!(code.contains("pub fn forward_prefill_batch(&mut self, tokens: &[u32])"));
        assert!(!code.contains('@'));
    }

    #[test]
    fn qwen2_and_mistral_reach_the_config() {
        let mut c = test_config();
        c.qkv_bias = true;
        c.sliding_window_size = Some(4096);
        c.dtype = DType::Q4_0;
        let code = generate_model_rs(&c).unwrap();
        assert!(code.contains("pub const FLAGS: u32 = 2;"));
        assert!(code.contains("pub const SLIDING_WINDOW_SIZE: usize = 4096;"));
        assert!(code.contains("pub const WDTYPE: u32 = 2;"));
    }

    #[test]
    fn unsupported_models_are_refused() {
        let mut c = test_config();
        c.dtype = DType::F32;
        assert!(matches!(generate_model_rs(&c), Err(HipCodegenError::Unsupported(_))));
        let mut c = test_config();
        c.head_dim = 256;
        assert!(matches!(generate_model_rs(&c), Err(HipCodegenError::Unsupported(_))));
    }

    #[test]
    fn project_files_are_written() {
        let dir = tempfile::tempdir().unwrap();
        let mut graph = Graph::new("test");
        graph.config = Some(test_config());
        generate_hip_project(&graph, dir.path(), "Test Model").unwrap();
        for f in ["Cargo.toml", "build.rs", "src/model.rs", "src/main.rs"] {
            assert!(dir.path().join(f).exists(), "{f} missing");
        }
        let cargo = std::fs::read_to_string(dir.path().join("Cargo.toml")).unwrap();
        assert!(cargo.contains("name = \"test-model\""));
        let main = std::fs::read_to_string(dir.path().join("src/main.rs")).unwrap();
        assert!(main.contains("--repeat-penalty") && main.contains("0xdeadbeef12345678"));
        assert!(!main.contains('@'));
    }

    #[test]
    fn missing_config_is_an_error() {
        let graph = Graph::new("empty");
        let dir = tempfile::tempdir().unwrap();
        assert!(matches!(generate_hip_project(&graph, dir.path(), "x"), Err(HipCodegenError::MissingConfig)));
    }
}
