//! `bpe_tokenizer` over the C ABI (`coeus_bpe_*` in include/coeus.h): the same traits and plugin id
//! as `plugins/tokenizer-bpe`.  Source only, like the rest of this crate (no Rust toolchain where
//! the library is built).  Results equal the Rust crate's token for token; the one convention is
//! in `train`: among equally frequent pairs the library merges the smallest pair in byte order,
//! where the Rust crate's choice follows its HashMap's random seed.
use rustllm_core::core::plugin::{Plugin, PluginCapabilities, TokenizerPlugin};
use rustllm_core::core::tokenizer::{StringToken, Token, TokenIterator, Tokenizer, VocabularyTokenizer};
use rustllm_core::core::traits::{Identity, Versioned};
use rustllm_core::foundation::{error::{invalid_input, Result},
                               types::{TokenId, Version, VocabSize}};
use std::borrow::Cow;
use std::ffi::CStr;
use std::os::raw::{c_char, c_int};

#[repr(C)] pub struct CoeusBpe { _private: [u8; 0] }

#[link(name = "coeus_mi355x")]
extern "C" {
    fn coeus_last_error() -> *const c_char;
    fn coeus_bpe_create(out: *mut *mut CoeusBpe) -> c_int;
    fn coeus_bpe_destroy(t: *mut CoeusBpe);
    fn coeus_bpe_train(t: *mut CoeusBpe, texts: *const *const c_char, lens: *const u64,
                       n_texts: u64, num_merges: u64) -> c_int;
    fn coeus_bpe_tokenize(t: *const CoeusBpe, text: *const c_char, len: u64, ids: *mut u64,
                          ids_cap: u64, n_tokens: *mut u64, pieces: *mut c_char, pieces_cap: u64,
                          offsets: *mut u64, pieces_len: *mut u64) -> c_int;
    fn coeus_bpe_decode(pieces: *const c_char, offsets: *const u64, n_tokens: u64, out: *mut c_char,
                        cap: u64, len: *mut u64) -> c_int;
    fn coeus_bpe_vocab_size(t: *const CoeusBpe) -> u64;
    fn coeus_bpe_add_token(t: *mut CoeusBpe, token: *const c_char, len: u64, id_out: *mut u64) -> c_int;
    fn coeus_bpe_remove_token(t: *mut CoeusBpe, token: *const c_char, len: u64) -> c_int;
    fn coeus_bpe_id_from_token(t: *const CoeusBpe, token: *const c_char, len: u64, id_out: *mut u64,
                               found: *mut c_int) -> c_int;
    fn coeus_bpe_token_from_id(t: *const CoeusBpe, id: u64, out: *mut c_char, cap: u64, len: *mut u64,
                               found: *mut c_int) -> c_int;
}

fn check(rc: c_int) -> Result<()> {
    if rc == 0 { return Ok(()); }
    Err(invalid_input(unsafe { CStr::from_ptr(coeus_last_error()) }.to_string_lossy().into_owned()))
}

#[derive(Debug, Default)] pub struct BpeTokenizerPlugin;
impl Identity for BpeTokenizerPlugin { fn id(&self) -> &str { "bpe_tokenizer" } }
impl Versioned for BpeTokenizerPlugin { fn version(&self) -> Version { Version::new(0, 1, 0) } }
impl Plugin for BpeTokenizerPlugin {
    fn capabilities(&self) -> PluginCapabilities {
        PluginCapabilities::standard().with_feature("tokenization").with_feature("bpe")
    }
}
impl TokenizerPlugin for BpeTokenizerPlugin {
    type Tokenizer = BpeTokenizer;
    fn create_tokenizer(&self) -> Result<Self::Tokenizer> { BpeTokenizer::new() }
}

#[derive(Debug)] pub struct BpeTokenizer { handle: *mut CoeusBpe }
unsafe impl Send for BpeTokenizer {}   // reads are thread-safe; mutation needs &mut self
unsafe impl Sync for BpeTokenizer {}
impl Drop for BpeTokenizer { fn drop(&mut self) { unsafe { coeus_bpe_destroy(self.handle) } } }

impl BpeTokenizer {
    pub fn new() -> Result<Self> {
        let mut h = std::ptr::null_mut();
        check(unsafe { coeus_bpe_create(&mut h) })?;
        Ok(Self { handle: h })
    }
    pub fn train(&mut self, corpus: &[&str], num_merges: usize) -> Result<()> {
        let ptrs: Vec<*const c_char> = corpus.iter().map(|s| s.as_ptr().cast()).collect();
        let lens: Vec<u64> = corpus.iter().map(|s| s.len() as u64).collect();
        check(unsafe { coeus_bpe_train(self.handle, ptrs.as_ptr(), lens.as_ptr(), corpus.len() as u64,
                                       num_merges as u64) })
    }
    /// The ids alone, widened to what `ForwardModel::forward` takes.
    pub fn encode(&self, text: &str) -> Result<Vec<usize>> {
        let (mut n, mut nb) = (0u64, 0u64);
        let p = text.as_ptr().cast();
        check(unsafe { coeus_bpe_tokenize(self.handle, p, text.len() as u64, std::ptr::null_mut(), 0, &mut n,
                                          std::ptr::null_mut(), 0, std::ptr::null_mut(), &mut nb) })?;
        let mut ids = vec![0u64; n as usize];
        check(unsafe { coeus_bpe_tokenize(self.handle, p, text.len() as u64, ids.as_mut_ptr(), n, &mut n,
                                          std::ptr::null_mut(), 0, std::ptr::null_mut(), &mut nb) })?;
        Ok(ids.into_iter().map(|i| i as usize).collect())
    }
}

impl Tokenizer for BpeTokenizer {
    type Token = StringToken;
    type Error = std::io::Error;

    fn tokenize<'a>(&self, input: Cow<'a, str>) -> TokenIterator<'a, Self::Token> {
        let (mut n, mut nb) = (0u64, 0u64);
        let (p, len) = (input.as_ptr().cast(), input.len() as u64);
        // a &str is valid UTF-8, the only input the library rejects: the calls cannot fail
        unsafe { coeus_bpe_tokenize(self.handle, p, len, std::ptr::null_mut(), 0, &mut n,
                                    std::ptr::null_mut(), 0, std::ptr::null_mut(), &mut nb) };
        let mut ids = vec![0u64; n as usize];
        let mut offs = vec![0u64; n as usize + 1];
        let mut bytes = vec![0u8; nb as usize];
        unsafe { coeus_bpe_tokenize(self.handle, p, len, ids.as_mut_ptr(), n, &mut n,
                                    bytes.as_mut_ptr().cast(), nb, offs.as_mut_ptr(), &mut nb) };
        let tokens: Vec<StringToken> = (0..n as usize).map(|i| {
            let s = String::from_utf8_lossy(&bytes[offs[i] as usize..offs[i + 1] as usize]).into_owned();
            StringToken::with_id(s, ids[i] as TokenId)
        }).collect();
        Box::new(tokens.into_iter())
    }

    fn decode<I>(&self, tokens: I) -> Result<String> where I: IntoIterator<Item = Self::Token> {
        let (mut bytes, mut offs) = (Vec::<u8>::new(), vec![0u64]);
        for t in tokens {
            if let Some(s) = t.as_str() { bytes.extend_from_slice(s.as_bytes()); }
            offs.push(bytes.len() as u64);
        }
        let n = offs.len() as u64 - 1;
        let mut len = 0u64;
        check(unsafe { coeus_bpe_decode(bytes.as_ptr().cast(), offs.as_ptr(), n, std::ptr::null_mut(), 0, &mut len) })?;
        let mut out = vec![0u8; len as usize];
        check(unsafe { coeus_bpe_decode(bytes.as_ptr().cast(), offs.as_ptr(), n, out.as_mut_ptr().cast(), len, &mut len) })?;
        Ok(String::from_utf8_lossy(&out).into_owned())
    }

    fn vocab_size(&self) -> VocabSize { unsafe { coeus_bpe_vocab_size(self.handle) as VocabSize } }
    fn name(&self) -> &str { "bpe_tokenizer" }
}

impl VocabularyTokenizer for BpeTokenizer {
    fn add_token(&mut self, token: &str) -> Result<TokenId> {
        let mut id = 0u64;
        check(unsafe { coeus_bpe_add_token(self.handle, token.as_ptr().cast(), token.len() as u64, &mut id) })?;
        Ok(id as TokenId)
    }
    fn remove_token(&mut self, token: &str) -> Result<()> {
        check(unsafe { coeus_bpe_remove_token(self.handle, token.as_ptr().cast(), token.len() as u64) })
    }
    fn contains_token(&self, token: &str) -> bool { self.id_from_token(token).is_some() }
    fn token_from_id(&self, id: TokenId) -> Option<String> {
        let (mut len, mut found) = (0u64, 0 as c_int);
        unsafe { coeus_bpe_token_from_id(self.handle, id as u64, std::ptr::null_mut(), 0, &mut len, &mut found) };
        if found == 0 { return None; }
        let mut out = vec![0u8; len as usize];
        unsafe { coeus_bpe_token_from_id(self.handle, id as u64, out.as_mut_ptr().cast(), len, &mut len, &mut found) };
        Some(String::from_utf8_lossy(&out).into_owned())
    }
    fn id_from_token(&self, token: &str) -> Option<TokenId> {
        let (mut id, mut found) = (0u64, 0 as c_int);
        unsafe { coeus_bpe_id_from_token(self.handle, token.as_ptr().cast(), token.len() as u64, &mut id, &mut found) };
        if found != 0 { Some(id as TokenId) } else { None }
    }
}
