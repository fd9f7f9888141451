//! Eclat backend for AMD MI355X (gfx950) -- binds `libeclat_hip` to the backend traits.
//!
//! SOURCE ONLY: the pipeline that produced this crate has no Rust toolchain; it has never been
//! compiled or run.  It shows which trait method each C entry point serves.
//!
//! The AST is serialised to the s-expression text `eh_program_compile` reads (one form per
//! `AstNode` variant, see `ser.rs`); rendering, hiprtc compilation, caching of code objects
//! and launching all happen behind the C ABI.

mod ffi;
mod ser;

use std::any::Any;
use std::collections::HashMap;
use std::ffi::{CStr, CString};
use std::sync::{Arc, Mutex, OnceLock};

use eclat::ast::{AstNode, DType};
use eclat::backend::device::{BackendRegistry, DeviceError, ProgramBuffer};
use eclat::backend::global::DeviceKind;
use eclat::backend::renderer::Renderer;
use eclat::backend::traits::{
    Buffer, Compiler, Device, DeviceFeature, DeviceInstruction, DeviceProfile, DeviceType, Kernel, KernelConfig,
    MatrixCapability, OpKind, SimdCapability,
};
use eclat::backend::KernelSignature;

type DynErr = Box<dyn std::error::Error + Send + Sync>;

/// The one place this crate aborts a caller: trait methods that return no `Result`.
fn panic_with(what: &str, why: &str) -> ! { std::panic::panic_any(format!("{what}: {why}")) }

fn check(code: i32) -> Result<(), DynErr> {
    if code == 0 { Ok(()) } else { Err(ffi::last_error().into()) }
}

struct DeviceHandle { raw: *mut ffi::eh_device }
unsafe impl Send for DeviceHandle {}
unsafe impl Sync for DeviceHandle {}
impl Drop for DeviceHandle { fn drop(&mut self) { unsafe { ffi::eh_device_close(self.raw); } } }

/// One opened GPU; clones share the handle, which closes when the last clone (a device, a
/// buffer or a kernel holds one each) is dropped.
#[derive(Clone)]
pub struct HipDevice { handle: Arc<DeviceHandle> }

impl HipDevice {
    pub fn open(index: usize) -> Result<Self, DynErr> {
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::eh_device_open(index as i32, &mut raw) })?;
        Ok(Self { handle: Arc::new(DeviceHandle { raw }) })
    }
    fn raw(&self) -> *mut ffi::eh_device { self.handle.raw }
    fn props(&self) -> Option<ffi::eh_device_props> {
        let mut p = std::mem::MaybeUninit::<ffi::eh_device_props>::zeroed();
        if unsafe { ffi::eh_device_get_props(self.raw(), p.as_mut_ptr()) } != 0 { return None; }
        Some(unsafe { p.assume_init() })
    }
}

/// `Device` (src/backend/traits.rs:273-306).  The profile describes gfx950 as the library
/// reports it; the AST-level parallelisation and matrix features are declined on purpose:
/// this backend takes the kernels as lowered (sequential `Range` nests) and picks the
/// work-item mapping, LDS staging and MFMA tiling itself while rendering.
impl Device for HipDevice {
    fn is_available() -> bool {
        let mut n = 0;
        unsafe { ffi::eh_device_count(&mut n) == 0 && n > 0 }
    }
    fn profile(&self) -> DeviceProfile {
        let (cus, wave, max_wg, lds) = match self.props() {
            Some(p) => (p.compute_units as usize, p.warp_size as usize, p.max_work_group_size as usize, p.local_memory_size),
            None => (256, 64, 1024, 160 * 1024),
        };
        let mut simd = Vec::new();
        for op in [OpKind::Add, OpKind::Mul, OpKind::Fma, OpKind::Compare, OpKind::Load, OpKind::Store] {
            simd.push(SimdCapability::new(DType::F32, op, 4));      // 16-byte global accesses
        }
        DeviceProfile {
            device_type: DeviceType::DiscreteGpu,
            compute_units: cus,
            max_work_group_size: max_wg,
            preferred_work_group_size_range: (wave, 256),
            local_memory_size: lds,
            warp_size: wave,
            preferred_tile_sizes: vec![16, 32, 64, 128, 256],
            simd_capabilities: simd,
            // v_mfma_f32_32x32x2_f32 and v_mfma_f32_16x16x4_f32
            matrix_capabilities: vec![MatrixCapability::new(DType::F32, DType::F32, 32, 32, 2),
                                      MatrixCapability::new(DType::F32, DType::F32, 16, 16, 4)],
        }
    }
    fn supports_feature(&self, feature: DeviceFeature) -> bool {
        match feature {
            DeviceFeature::FastMath | DeviceFeature::HalfPrecision | DeviceFeature::DoublePrecision
            | DeviceFeature::LocalMemory | DeviceFeature::AtomicOperations | DeviceFeature::SubgroupOperations => true,
            DeviceFeature::ParallelKernel | DeviceFeature::MatrixOperations => false,
        }
    }
    fn supports_instruction(&self, instruction: DeviceInstruction) -> bool {
        match instruction {
            DeviceInstruction::Fma | DeviceInstruction::Rsqrt | DeviceInstruction::AtomicAddFloat
            | DeviceInstruction::NativeDiv | DeviceInstruction::NativeExpLog => true,
        }
    }
}

pub struct HipBuffer { raw: *mut ffi::eh_buffer, dev: HipDevice, shape: Vec<usize>, dtype: DType, bytes: usize }
unsafe impl Send for HipBuffer {}
unsafe impl Sync for HipBuffer {}
impl Drop for HipBuffer { fn drop(&mut self) { unsafe { ffi::eh_buffer_release(self.raw); } } }

impl HipBuffer {
    fn allocate(dev: &HipDevice, shape: Vec<usize>, dtype: DType) -> Result<Self, DynErr> {
        let bytes = shape.iter().product::<usize>() * dtype.size_in_bytes();
        let mut raw = std::ptr::null_mut();
        check(unsafe { ffi::eh_buffer_alloc(dev.raw(), bytes, &mut raw) })?;   // zero-filled
        Ok(Self { raw, dev: dev.clone(), shape, dtype, bytes })
    }
}

impl Buffer for HipBuffer {
    fn shape(&self) -> &[usize] { &self.shape }
    fn dtype(&self) -> DType { self.dtype.clone() }
    fn byte_len(&self) -> usize { self.bytes }
    fn read_to_host(&self) -> Result<Vec<u8>, DynErr> {
        let mut v = vec![0u8; self.bytes];
        check(unsafe { ffi::eh_buffer_read(self.raw, v.as_mut_ptr().cast(), self.bytes) })?;
        Ok(v)
    }
    fn write_from_host(&mut self, data: &[u8]) -> Result<(), DynErr> {
        // the library rejects a length different from byte_len(), as CBuffer does
        check(unsafe { ffi::eh_buffer_write(self.raw, data.as_ptr().cast(), data.len()) })
    }
    fn clone_buffer(&self) -> Box<dyn Buffer> {
        // The trait has no error path here (CBuffer clones a Vec, which aborts when memory runs
        // out): a failed allocation or device copy ends in a panic that carries the library's
        // message, never in a buffer that silently holds something else.
        let b = HipBuffer::allocate(&self.dev, self.shape.clone(), self.dtype.clone())
            .unwrap_or_else(|e| panic_with("clone_buffer: allocation failed", &e.to_string()));
        if let Err(e) = check(unsafe { ffi::eh_buffer_copy(b.raw, self.raw) }) {
            panic_with("clone_buffer: device copy failed", &e.to_string());
        }
        Box::new(b)
    }
    fn as_any(&self) -> &dyn Any { self }
    fn as_any_mut(&mut self) -> &mut dyn Any { self }
}

enum Loaded { Program(*mut ffi::eh_program), Module(*mut ffi::eh_module) }

/// `ast_text` is kept for kernels compiled from an AST, `blob` (the gfx950 code object) for kernels
/// loaded through `Compiler::compile`: either is what `clone_kernel` builds the copy from.
pub struct HipKernel { loaded: Loaded, config: KernelConfig, ast_text: Option<Arc<String>>, blob: Option<Arc<Vec<u8>>>, dev: HipDevice }
unsafe impl Send for HipKernel {}
unsafe impl Sync for HipKernel {}
impl Drop for HipKernel {
    fn drop(&mut self) {
        unsafe {
            match self.loaded {
                Loaded::Program(p) => { ffi::eh_program_release(p); }
                Loaded::Module(m) => { ffi::eh_module_release(m); }
            }
        }
    }
}

fn raw_buffers(bufs: &[&dyn Buffer]) -> Vec<*mut ffi::eh_buffer> {
    bufs.iter().map(|b| b.as_any().downcast_ref::<HipBuffer>().expect("buffer is not a HipBuffer").raw).collect()
}

impl Kernel for HipKernel {
    fn clone_kernel(&self) -> Box<dyn Kernel> {
        // from the AST text (the library's code-object cache makes the recompile a lookup), or, for a
        // kernel that came in as source through `Compiler::compile`, from its code object
        let made = match (&self.ast_text, &self.blob) {
            (Some(text), _) => compile_text(&self.dev, text.clone(), self.config.clone()),
            (None, Some(blob)) => load_blob(&self.dev, blob.clone(), self.config.clone()),
            (None, None) => Err("kernel holds neither its AST nor its code object".into()),
        };
        Box::new(made.unwrap_or_else(|e| panic_with("clone_kernel", &e.to_string())))
    }
    fn config(&self) -> &KernelConfig { &self.config }
    fn device_kind(&self) -> DeviceKind { DeviceKind::Hip }
    fn execute(&self, inputs: &[&dyn Buffer], outputs: &mut [&mut dyn Buffer]) -> Result<(), DynErr> {
        let ins = raw_buffers(inputs);
        let outs: Vec<_> = outputs.iter().map(|b| b.as_any().downcast_ref::<HipBuffer>()
            .expect("buffer is not a HipBuffer").raw).collect();
        match self.loaded {
            Loaded::Program(p) => check(unsafe {
                ffi::eh_program_execute_positional(p, ins.as_ptr(), ins.len() as i32, outs.as_ptr(), outs.len() as i32, wait_per_launch())
            }),
            Loaded::Module(_) => {
                let g = self.config.global_work_size;
                let l = self.config.local_work_size.unwrap_or([1, 1, 1]);
                self.execute_with_sizes(inputs, outputs, g, l)
            }
        }
    }
    fn execute_with_sizes(&self, inputs: &[&dyn Buffer], outputs: &mut [&mut dyn Buffer],
                          grid_size: [usize; 3], local_size: [usize; 3]) -> Result<(), DynErr> {
        // `grid_size` is the global size here; the library wants workgroup counts
        let Loaded::Module(m) = self.loaded else { return self.execute(inputs, outputs); };
        let mut args = raw_buffers(inputs);
        args.extend(outputs.iter().map(|b| b.as_any().downcast_ref::<HipBuffer>().expect("not a HipBuffer").raw));
        let block = local_size.map(|v| v.max(1) as u32);
        let grid = [0, 1, 2].map(|i| (grid_size[i].max(1) as u32).div_ceil(block[i]));
        check(unsafe { ffi::eh_module_launch(m, grid.as_ptr(), block.as_ptr(), 0, args.as_ptr(), args.len() as i32, 1) })
    }
    fn as_any(&self) -> &dyn Any { self }
    // One AST kernel may become several launches (a reduce cut over workgroups, a split-K
    // contraction and its summing launch), each with its own entry point, grid and block; the
    // core's disk cache (src/backend/global.rs:283-345) stores one blob under the AST kernel's
    // name with a 1x1x1 dispatch and could not restore that.  The library keeps its own verified
    // cache of code objects on disk ($HARP_CACHE_DIR/code_objects/gfx950), keyed by the generated
    // source, so nothing is lost by declining the core's.
    fn supports_binary_cache(&self) -> bool { false }
    fn get_binary(&self) -> Option<Vec<u8>> { None }
}

fn compile_text(dev: &HipDevice, text: Arc<String>, config: KernelConfig) -> Result<HipKernel, DynErr> {
    let c = CString::new(text.as_str())?;
    let mut raw = std::ptr::null_mut();
    check(unsafe { ffi::eh_program_compile(dev.raw(), c.as_ptr(), std::ptr::null(), &mut raw) })?;
    Ok(HipKernel { loaded: Loaded::Program(raw), config, ast_text: Some(text), blob: None, dev: dev.clone() })
}

fn load_blob(dev: &HipDevice, blob: Arc<Vec<u8>>, config: KernelConfig) -> Result<HipKernel, DynErr> {
    let entry = CString::new(config.entry_point.as_str())?;
    let mut raw = std::ptr::null_mut();
    check(unsafe { ffi::eh_module_load(dev.raw(), blob.as_ptr().cast(), blob.len(), entry.as_ptr(), &mut raw) })?;
    Ok(HipKernel { loaded: Loaded::Module(raw), config, ast_text: None, blob: Some(blob), dev: dev.clone() })
}

/// `Renderer` (src/backend/renderer.rs:20-35): AST -> HIP C, no device involved.  The text is
/// every launch's translation unit in launch order; dispatch sizes come with the plan
/// (`eh_plan_launch`), not from the AST's grid fields.
///
/// `CLikeRenderer` and `KernelSourceRenderer` (src/backend/renderer.rs:69-159,
/// src/backend/pipeline.rs:27-33) are deliberately NOT implemented, so the generic
/// `Pipeline<R, Dev, Comp>` (pipeline.rs:135-216) cannot be instantiated with this renderer.
/// That pipeline renders one translation unit, takes the first kernel's name as the entry point
/// and the AST's own grid and thread-group fields as the dispatch (1x1x1 for a lowered kernel),
/// and compiles exactly that.  Here one AST kernel becomes one or several launches with entry
/// points, grids, workgroup sizes and sometimes scratch buffers that only the plan knows: fed
/// through the generic pipeline the code would be launched with the wrong entry and geometry.
/// `BackendRegistry::compile_ast` and `execute_program` below are the routes; both hand the AST
/// to the library, which plans, renders, compiles and launches as one unit.
#[derive(Default)]
pub struct HipRenderer { options: Option<String> }

impl Renderer for HipRenderer {
    type CodeRepr = String;
    type Option = String;          // "key=value,..." as `eh_render_program` takes it
    fn render(&self, program: &AstNode) -> String {
        let text = match ser::to_text(program) {
            Ok(t) => t,
            Err(e) => return format!("/* {e} */"),
        };
        let Ok(text) = CString::new(text) else { return String::new(); };
        let opts = self.options.as_ref().and_then(|o| CString::new(o.as_str()).ok());
        let mut plan = std::ptr::null_mut();
        let optr = opts.as_ref().map_or(std::ptr::null(), |o| o.as_ptr());
        if unsafe { ffi::eh_render_program(text.as_ptr(), optr, &mut plan) } != 0 {
            return format!("/* {} */", ffi::last_error());
        }
        let mut out = String::new();
        let mut n = 0;
        unsafe {
            ffi::eh_plan_num_launches(plan, &mut n);
            for i in 0..n {
                let mut info = std::mem::MaybeUninit::<ffi::eh_launch_info>::zeroed();
                if ffi::eh_plan_launch(plan, i, info.as_mut_ptr()) == 0 {
                    out.push_str(&std::ffi::CStr::from_ptr(info.assume_init().source).to_string_lossy());
                    out.push('\n');
                }
            }
            ffi::eh_plan_release(plan);
        }
        out
    }
    fn is_available(&self) -> bool { true }     // rendering needs no GPU
    fn with_option(&mut self, option: String) { self.options = Some(option); }
}

/// `Compiler` (src/backend/traits.rs:592-607): HIP C source -> gfx950 code object with hiprtc,
/// loaded as one entry point; `config` carries the entry name and the dispatch sizes.
pub struct HipCompiler;

impl Compiler for HipCompiler {
    type Dev = HipDevice;
    type Kernel = HipKernel;
    type Error = std::io::Error;
    fn new() -> Self { HipCompiler }
    fn compile(&self, device: &HipDevice, source: &str, config: KernelConfig) -> Result<HipKernel, std::io::Error> {
        let err = |m: String| std::io::Error::new(std::io::ErrorKind::Other, m);
        let src = CString::new(source).map_err(|e| err(e.to_string()))?;
        let entry = CString::new(config.entry_point.as_str()).map_err(|e| err(e.to_string()))?;
        let (mut blob, mut len) = (std::ptr::null_mut(), 0usize);
        if unsafe { ffi::eh_compile_source(src.as_ptr(), std::ptr::null(), &mut blob, &mut len) } != 0 {
            return Err(err(ffi::last_error()));
        }
        let _ = entry;
        // the code object is kept beside the loaded module, so that the kernel can be cloned
        let owned = Arc::new(unsafe { std::slice::from_raw_parts(blob as *const u8, len) }.to_vec());
        unsafe { ffi::eh_free(blob); }
        load_blob(device, owned, config).map_err(|e| err(e.to_string()))
    }
}

struct HipBackendRegistry;

fn device_of(device: &dyn Any) -> Result<&HipDevice, DeviceError> {
    device.downcast_ref::<HipDevice>()
        .ok_or_else(|| DeviceError::InitializationError("Invalid device type: expected HipDevice".into()))
}

impl BackendRegistry for HipBackendRegistry {
    fn kind(&self) -> DeviceKind { DeviceKind::Hip }
    fn name(&self) -> &str { "HIP (gfx950)" }
    fn is_available(&self) -> bool {
        let mut n = 0;
        unsafe { ffi::eh_device_count(&mut n) == 0 && n > 0 }
    }
    fn create_device(&self, index: usize) -> Result<Arc<dyn Any + Send + Sync>, DeviceError> {
        HipDevice::open(index).map(|d| Arc::new(d) as Arc<dyn Any + Send + Sync>)
            .map_err(|e| DeviceError::InitializationError(e.to_string()))
    }
    fn list_devices(&self) -> Vec<String> {
        let mut n = 0;
        unsafe { ffi::eh_device_count(&mut n); }
        (0..n).map(|i| format!("hip:{i}")).collect()
    }
    fn supports_runtime(&self) -> bool { true }
    fn allocate_buffer(&self, device: &dyn Any, shape: Vec<usize>, dtype: DType) -> Result<Box<dyn Buffer>, DeviceError> {
        let dev = device_of(device)?;
        HipBuffer::allocate(dev, shape, dtype).map(|b| Box::new(b) as Box<dyn Buffer>)
            .map_err(|e| DeviceError::InitializationError(format!("Failed to allocate HIP buffer: {e}")))
    }
    fn compile_ast(&self, device: &dyn Any, program: AstNode, _signature: KernelSignature)
                   -> Result<Box<dyn Kernel>, DeviceError> {
        let dev = device_of(device)?;
        let entry = ser::first_kernel_name(&program).unwrap_or_else(|| "kernel".to_string());
        let text = Arc::new(ser::to_text(&program).map_err(DeviceError::InitializationError)?);
        compile_text(dev, text, KernelConfig::new(entry)).map(|k| Box::new(k) as Box<dyn Kernel>)
            .map_err(|e| DeviceError::InitializationError(format!("Failed to compile AST: {e}")))
    }
    // declined, with the kernels': see HipKernel::supports_binary_cache
    fn supports_binary_cache(&self) -> bool { false }

    /// The whole lowered Program at once (the hook `core-edits.patch` adds to the trait and to
    /// `execute_graph`): the library fuses kernels over the same index space into one launch,
    /// keeps temporaries that never leave a launch out of memory and runs contractions on MFMA
    /// with their elementwise consumers as epilogue.  Results are those of the per-kernel path.
    /// `buffers` holds the inputs by name; outputs (the roots' buffers) are allocated here and
    /// inserted; temporaries stay inside the compiled program.
    fn execute_program(&self, device: &dyn Any, kernels: &[AstNode], table: &[ProgramBuffer],
                       buffers: &mut HashMap<String, Box<dyn Buffer>>) -> Option<Result<(), DeviceError>> {
        Some(run_program(device, kernels, table, buffers))
    }
}

struct ProgramHandle { raw: *mut ffi::eh_program, _dev: HipDevice }
unsafe impl Send for ProgramHandle {}
unsafe impl Sync for ProgramHandle {}
impl Drop for ProgramHandle { fn drop(&mut self) { unsafe { ffi::eh_program_release(self.raw); } } }

/// Compiled programs by (device, program text): planning and module loading happen once per
/// distinct program, as the core's kernel cache does per kernel (src/backend/cache/store.rs:116-168;
/// same capacity, oldest entry out).
fn program_cache() -> &'static Mutex<Vec<((usize, String), Arc<ProgramHandle>)>> {
    static CACHE: OnceLock<Mutex<Vec<((usize, String), Arc<ProgramHandle>)>>> = OnceLock::new();
    CACHE.get_or_init(|| Mutex::new(Vec::new()))
}

fn compiled_program(dev: &HipDevice, text: String) -> Result<Arc<ProgramHandle>, DeviceError> {
    let key = (dev.raw() as usize, text);
    let mut cache = program_cache().lock().unwrap();
    if let Some(pos) = cache.iter().position(|(k, _)| *k == key) {
        let hit = cache.remove(pos);
        let prog = hit.1.clone();
        cache.push(hit);                                   // most recently used last
        return Ok(prog);
    }
    let c = CString::new(key.1.as_str()).map_err(|e| DeviceError::InitializationError(e.to_string()))?;
    let mut raw = std::ptr::null_mut();
    if unsafe { ffi::eh_program_compile(dev.raw(), c.as_ptr(), std::ptr::null(), &mut raw) } != 0 {
        return Err(DeviceError::InitializationError(format!("Failed to compile program: {}", ffi::last_error())));
    }
    let prog = Arc::new(ProgramHandle { raw, _dev: dev.clone() });
    if cache.len() >= 1024 { cache.remove(0); }
    cache.push((key, prog.clone()));
    Ok(prog)
}

fn run_program(device: &dyn Any, kernels: &[AstNode], table: &[ProgramBuffer],
               buffers: &mut HashMap<String, Box<dyn Buffer>>) -> Result<(), DeviceError> {
    let err = |m: String| DeviceError::InitializationError(m);
    let dev = device_of(device)?;
    let prog = compiled_program(dev, ser::program_text(kernels, table).map_err(err)?)?;
    let mut n = 0;
    if unsafe { ffi::eh_program_num_buffers(prog.raw, &mut n) } != 0 { return Err(err(ffi::last_error())); }
    // the library's table: the caller's entries in their order, then scratch temps of its own
    let mut raws: Vec<*mut ffi::eh_buffer> = Vec::with_capacity(n as usize);
    for i in 0..n {
        let (mut name, mut role) = (std::ptr::null(), std::ptr::null());
        let (mut bytes, mut elided) = (0usize, 0);
        if unsafe { ffi::eh_program_buffer(prog.raw, i, &mut name, &mut role, &mut bytes, &mut elided) } != 0 {
            return Err(err(ffi::last_error()));
        }
        let name = unsafe { CStr::from_ptr(name) }.to_string_lossy().into_owned();
        let role = unsafe { CStr::from_ptr(role) }.to_string_lossy().into_owned();
        if elided != 0 { raws.push(std::ptr::null_mut()); continue; }
        if !buffers.contains_key(&name) {
            if role != "output" { raws.push(std::ptr::null_mut()); continue; }    // a temp: the program keeps it
            let info = table.iter().find(|b| b.name == name)
                .ok_or_else(|| err(format!("output '{name}' is missing from the buffer table")))?;
            let out = HipBuffer::allocate(dev, info.shape.clone(), info.dtype.clone())
                .map_err(|e| err(format!("Failed to allocate buffer '{name}': {e}")))?;
            buffers.insert(name.clone(), Box::new(out));
        }
        let b = buffers.get(&name).unwrap().as_any().downcast_ref::<HipBuffer>()
            .ok_or_else(|| err(format!("buffer '{name}' is not a HipBuffer")))?;
        raws.push(b.raw);
    }
    if unsafe { ffi::eh_program_execute(prog.raw, raws.as_ptr(), n, wait_per_launch()) } != 0 { return Err(err(ffi::last_error())); }
    Ok(())
}

/// Launches are queued on the device's stream and not waited for: every read of a buffer
/// (`Buffer::read_to_host` waits for the stream), every copy and every reuse of released memory is
/// ordered behind them there, so a caller cannot see the difference except in time -- and in where
/// a device fault is reported (at the next read instead of at `execute`).  ECLAT_HIP_SYNC=1 makes
/// every `execute` wait, as the reference's own backends do.
fn wait_per_launch() -> i32 {
    static WAIT: OnceLock<i32> = OnceLock::new();
    *WAIT.get_or_init(|| if std::env::var("ECLAT_HIP_SYNC").map(|v| v == "1").unwrap_or(false) { 1 } else { 0 })
}

/// Registers the backend (called at program start when the crate is linked).
pub fn init() { eclat::backend::register_backend(Box::new(HipBackendRegistry)); }

#[ctor::ctor]
fn auto_init() { init(); }
