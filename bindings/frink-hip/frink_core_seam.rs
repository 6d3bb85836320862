// What crates/frink-core gains for the HIP backend, as the fragments a maintainer pastes where the
// CUDA arms already are.  Not a compilation unit: each fragment names the file and the place it goes.
// (Never compiled in the library's repository, whose image has no Rust toolchain.)

// ---- crates/frink-core/Cargo.toml ----
//   [dependencies]  frink-hip = { workspace = true, optional = true }
//   [features]      hip = ["dep:frink-hip", "frink-hip/hip"]

// ---- crates/frink-core/src/weight_matrix/gpu_backend.rs, beside `pub struct Cuda;` ----
pub struct Hip;

impl BackendCaps for Hip {
    const ID: Backend = Backend::Hip; // a new kernel_registry::Backend variant
    const NAME: &'static str = "HIP";
    const GEMM_FALLBACK: &'static str = "HIP N x matvec batch";
    fn matvec_kernel(kind: QuantKind) -> Option<&'static str> {
        // the kinds libfrink_hip has kernels for: frk_hip_matvec_kernel() answers the same
        matches!(
            kind,
            QuantKind::Q4_0 | QuantKind::Q5_0 | QuantKind::Q8_0 | QuantKind::Q4K | QuantKind::Q5K | QuantKind::Q6K
                | QuantKind::IQ4XS | QuantKind::Mxfp4Gguf
        )
        .then(|| kind.name())
    }
    fn gemm_supported(kind: QuantKind) -> bool {
        matches!(
            kind,
            QuantKind::Q4_0 | QuantKind::Q5_0 | QuantKind::Q8_0 | QuantKind::Q4K | QuantKind::Q5K | QuantKind::Q6K
                | QuantKind::IQ4XS | QuantKind::Mxfp4Gguf
        )
    }
}

#[cfg(feature = "hip")]
impl BackendDispatch for Hip {
    const MATVEC_FALLBACK: &'static str = "CPU";
    fn dense_enabled() -> bool {
        frink_hip::dense_enabled() // FRINK_HIP, the grammar of env_or_probe
    }
    fn has_launch(kind: QuantKind) -> bool {
        frink_hip::kind_id(kind.name()).map_or(false, frink_hip::has_launch)
    }
    fn launch_matvec(kind: QuantKind, weights: &[u8], x: &[f32], rows: usize, row_bytes: usize)
        -> Option<Result<Vec<f32>, BackendError>> {
        let id = frink_hip::kind_id(kind.name())?; // None: no kernel for this kind
        Some(frink_hip::launch_matvec(id, weights, x, rows, row_bytes).map_err(|e| BackendError::new(e.message)))
    }
}

// one more row of the table (native backends before Vulkan, gpu_backend.rs:1008-1017)
macro_rules! gpu_backend_table { ($mac:path $(, $extra:tt)*) => { $mac! { [$($extra),*]
    (Cuda, "cuda", Cuda), (Metal, "metal", Metal), (Hip, "hip", Hip), (Vulkan, "vulkan", Vulkan), } }; }

// ---- crates/frink-core/src/weight_matrix.rs, beside `cuda_matvec_launch` (:1434-1457) ----
#[cfg(feature = "hip")]
impl WeightMatrix {
    pub fn hip_matvec_launch(&self) -> Option<frink_hip::MatvecLaunch<'_>> {
        let WeightMatrix::Quantized { data, rows, cols, kind } = self else { return None };
        let id = frink_hip::kind_id(kind.name())?;
        frink_hip::has_launch(id).then(|| frink_hip::MatvecLaunch {
            kind: id,
            weights: data.as_slice(),
            rows: *rows,
            row_bytes: self.block_bytes_per_row(*kind, *cols),
        })
    }
}

// ---- WeightMatrix::apply_gpu_multi_folded (:3586), after the CUDA arm ----
#[cfg(feature = "hip")]
if Hip::dense_enabled() {
    let mut launches = Vec::with_capacity(mats.len());
    for m in mats {
        assert_eq!(m.cols(), mats[0].cols());
        launches.push(m.hip_matvec_launch()?);
    }
    match frink_hip::launch_matvec_multi(x, &launches) {
        Ok(outs) => return Some(outs),
        Err(e) => eprintln!("frink: HIP multi-matvec failed, trying next backend: {e}"),
    }
}

// ---- WeightMatrix::apply_gpu_dense_ffn_swiglu (:3682), after the CUDA arm ----
#[cfg(feature = "hip")]
{
    if Hip::dense_enabled() {
        if let (Some(g), Some(u), Some(d)) = (gate.hip_matvec_launch(), up.hip_matvec_launch(), down.hip_matvec_launch()) {
            assert_eq!(gate.cols(), x.len());
            assert_eq!(up.cols(), x.len());
            assert_eq!(down.cols(), gate.rows());
            match frink_hip::launch_dense_ffn_swiglu(&g, &u, &d, x) {
                Ok(out) => return Some(out),
                Err(e) => eprintln!("frink: HIP dense FFN fuse failed, trying next: {e}"),
            }
        }
    }
}

// ---- WeightMatrix::apply_batch_with_acts (:2481) and apply_batch_pair_with_acts (:2447), where the CUDA arm
//      calls cuda_mul_mm_view ----
#[cfg(feature = "hip")]
if Hip::dense_enabled() && frink_hip::worth_a_gemm(batch) {
    if let WeightMatrix::Quantized { data, rows, cols, kind } = self {
        if let Some(id) = frink_hip::kind_id(kind.name()).filter(|&id| frink_hip::gemm_supported(id)) {
            let row_bytes = self.block_bytes_per_row(*kind, *cols);
            match frink_hip::launch_mul_mm(id, data.as_slice(), x_batch, *rows, *cols, batch, row_bytes) {
                Ok(out) => return out, // out[token * rows + row], the layout of :2310-2316
                Err(e) => eprintln!("frink: HIP mul_mm failed, falling back: {e}"),
            }
        }
    }
}
// (a resident prefill stack calls frink_hip::dev::gemm_pair for gate and up instead: one quantization of the batch)

// ---- crates/frink-models/src/decoder/ffn_batch.rs, Decoder::moe_ffn_batch (:343-434) ----
// Routing stays on the host (route_for_layer) or moves to frink_hip::dev::route_top_k_softmax; then, instead of
// the bucket / apply_batch / scatter-add loop, ONE call per layer on experts registered once as three stacked
// matrices (GGUF stores ffn_gate_exps / ffn_up_exps / ffn_down_exps that way):
#[cfg(feature = "hip")]
unsafe {
    frink_hip::dev::moe_ffn(&layer.gate_exps, &layer.up_exps, &layer.down_exps, n_experts, x_dev, batch, ids_dev,
                            weights_dev, k, out_dev, stream)?;
}
