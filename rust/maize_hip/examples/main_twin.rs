//! Twin of the reference's src/main.rs: the same 4096 x 4096 x 4096 bf16 problem and the same builder
//! chain, but the chain ends in a launch and a checked C instead of a printed PTX string.
use maize_hip::ffi::{maize_fill_uniform_bf16, MaizeGemmArgs};
use maize_hip::reference::{gemm_nn, ulp_distance};
use maize_hip::{new_hip_kernel, Ctx, Gfx, Layout, BF16};

fn fill(n: usize, seed: u64) -> Vec<BF16> {
    let mut v = vec![BF16(0); n];
    unsafe { maize_fill_uniform_bf16(v.as_mut_ptr() as *mut u16, n, seed, 0) };
    v
}

fn main() -> Result<(), Box<dyn std::error::Error>> {
    let (m, n, k) = (4096usize, 4096usize, 4096usize);
    let ctx = Ctx::new(0)?;
    let (a, b) = (fill(m * k, 0x5EED0001), fill(k * n, 0x5EED0002));
    let (da, db) = (ctx.upload(&a)?, ctx.upload(&b)?);
    let dc = ctx.malloc::<BF16>(m * n)?;
    let (amat, bmat, cmat) = (da.matrix(m as u32, k as u32), db.matrix(k as u32, n as u32), dc.matrix(m as u32, n as u32));

    // 1. the north-star entry: the library picks kernel and grid
    println!("dispatcher picks {}", ctx.gemm_select(amat, bmat, cmat, Layout::NN)?);
    ctx.gemm_bf16(amat, bmat, cmat, Layout::NN)?;
    ctx.sync()?;
    let c1 = dc.download()?;

    // 2. the reference's explicit chain: kernel -> launch bounds -> finalize -> compile(target) -> launch
    let kernel = new_hip_kernel("maize_gemm_bf16_mt256_nn").with_launch_bounds_2d((256, 1), None, None).finalize().compile(&Gfx::Gfx950, &ctx)?;
    let args = MaizeGemmArgs {
        a: amat.ptr as *const _, arows: amat.nrows, acols: amat.ncols,
        b: bmat.ptr as *const _, brows: bmat.nrows, bcols: bmat.ncols,
        c: cmat.ptr as *mut _, crows: cmat.nrows, ccols: cmat.ncols,
        stride_a: 0, stride_b: 0, stride_c: 0, batch: 1, layout: 0,
        workspace: std::ptr::null_mut(), ksplit: 0, reserved: 0,
        lda: 0, ldb: 0, ldc: 0, epi: 0, alpha: 0.0, beta: 0.0,
    };
    kernel.launch([256, 1, 1], &args)?; // persistent: any grid.x computes every tile
    ctx.sync()?;
    let c2 = dc.download()?;
    assert!(c1 == c2, "the two launch paths disagree");

    // 3. check 8 rows against the CPU twin
    let rows = [0usize, 1, 255, 256, 2047, 2048, 4094, 4095];
    let mut worst = 0u32;
    for &r in &rows {
        let want = gemm_nn(&a[r * k..(r + 1) * k], &b, 1, n, k);
        for j in 0..n {
            worst = worst.max(ulp_distance(c1[r * n + j], want[j]));
        }
    }
    println!("max bf16 ULP distance on {} sampled rows: {}", rows.len(), worst);
    Ok(())
}
