// x17ai_probe.cpp -- the measurement aids of include/x17ai_probe.h: a copy kernel, a matrix-core loop and a
// vector-issue loop, built and launched through the operator layer's kernel builder.  Nothing here is on the
// product path; the benchmark loads this library only for its calibration figures.
#include "../host/x17ai_host.hpp"
#include "../../../include/x17ai_probe.h"

#include <memory>
#include <string>

using namespace x17;

namespace {
	thread_local std::string g_error;
	int fail(std::string msg) { g_error = std::move(msg); return 1; }
	int fail_diag(char const *what, Diagnostics const &d) {
		std::string msg = std::string("failed to generate the ") + what + " kernel";
		for (auto const &x : d.list) if (x.is_error) { msg += "\n" + x.message; }
		return fail(std::move(msg));
	}
	int from_status(Status const &s) { return s.is_ok() ? 0 : fail(s.error->message); }

	struct Built { std::unique_ptr<HipKernel> kernel; std::vector<std::pair<std::string, size_t>> meta; };
	// source files sit beside this one: csrc/probes, reached from the kernel directory
	bool build(X17hDevice *dev, std::string const &name, std::string const &common, char const *source, char const *meta_source,
	           char const *what, Built &out) {
		Diagnostics diag;
		auto built = kernel_build::build(name, common, std::string("../probes/") + source, std::string("../probes/") + meta_source, diag);
		if (!built) { fail_diag(what, diag); return false; }
		auto meta = kernel_build::read_metadata_json(built->meta_json_path, diag);
		if (!meta) { fail_diag(what, diag); return false; }
		out.meta = *meta;
		if (dev != nullptr) {
			out.kernel = kernel_build::load_kernel(*dev->dev->stream, built->code_object_path, "kernel", 0, diag);
			if (!out.kernel) { fail_diag(what, diag); return false; }
		}
		return true;
	}
	size_t meta(Built const &b, char const *key) { auto v = kernel_build::meta_get(b.meta, key); return v ? *v : size_t(0); }

	// entries 0..27 are single instructions (X17_PROBE_OP = the index), the rest composite loops (X17_PROBE_OP = 100 + ...)
	char const *const VALU_OPS[] = {
		"v_fma_f32", "v_add_f32", "v_mul_f32", "v_xor_b32", "v_add_u32", "v_cvt_f32_i32", "v_rndne_f32", "v_max_f32", "v_max3_i32",
		"v_perm_b32", "v_cvt_pkrtz_f16_f32", "v_pk_mul_f16", "v_pk_fma_f16", "v_pk_add_f16", "v_med3_f32", "v_exp_f32", "v_rcp_f32",
		"v_log_f32", "v_permlane32_swap_b32", "s_add_u32", "v_lshl_add_u32", "v_add3_u32", "v_pack_b32_f16", "v_and_or_b32",
		"v_cndmask_b32", "v_cmp_lt_f32", "v_fmaak_f32", "v_mov_b32",
		"group: f16 mfma 32x32x16 (4 accumulators)", "group: i8 mfma 32x32x32 + 8 v_fma_f32", "group: i8 mfma 32x32x32 + 8 v_perm_b32",
		"group: i8 mfma 32x32x32 + 8 v_exp_f32", "group: i8 mfma 32x32x32 (dependent chain)",
		"group: attention step, vector + matrix instructions", "group: attention step, all instructions",
	};
	constexpr int N_SINGLE_OPS = 28;
	int probe_op_code(int index) { return index < N_SINGLE_OPS ? index : 100 + (index - N_SINGLE_OPS); }
	constexpr int N_VALU_OPS = int(sizeof VALU_OPS / sizeof VALU_OPS[0]);
}

struct X17pCopyProbe { std::shared_ptr<HipDevice> dev; Built b; };
struct X17pMfmaProbe { std::shared_ptr<HipDevice> dev; Built b; };
struct X17pValuProbe { std::shared_ptr<HipDevice> dev; Built b; };

extern "C" {

char const *x17p_last_error(void) { return g_error.c_str(); }

int x17p_copy_probe_new(X17hDevice *dev, X17pCopyProbe **out) {
	try {
		auto p = std::make_unique<X17pCopyProbe>();
		if (!build(dev, "copy_probe", "// copy probe\n", "copy_probe.hip", "copy_probe_meta.cpp", "copy probe", p->b)) return 1;
		if (dev != nullptr) p->dev = dev->dev;
		*out = p.release();
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
void x17p_copy_probe_free(X17pCopyProbe *p) { delete p; }
int x17p_copy_probe_launch(X17pCopyProbe *p, X17hTensor *src, X17hTensor *dst) {
	if (!p->b.kernel) return fail("copy probe was built without a device");
	if (src->t->bytes != dst->t->bytes || src->t->bytes % 16 != 0 || src->t->bytes / 16 > 0xFFFFFFFFull) return fail("copy probe needs equal sizes, multiple of 16 bytes");
	void *s = src->t->ptr, *d = dst->t->ptr;
	size_t n = src->t->bytes / 16;
	void *args[3] = {&s, &n, &d};
	size_t grid[3] = {meta(p->b, "BLOCKS"), 1, 1}, block[3] = {256, 1, 1};
	return from_status(p->b.kernel->launch(*p->dev->stream, grid, block, 0, args));
}

int x17p_mfma_probe_new(X17hDevice *dev, int kind, X17pMfmaProbe **out) {
	try {
		if (kind < 0 || kind > 2) return fail("mfma probe kind: 0 int8, 1 e4m3, 2 f16");
		auto p = std::make_unique<X17pMfmaProbe>();
		if (!build(dev, "mfma_probe-kind" + std::to_string(kind), "// matrix-core probe\n#define X17_PROBE_KIND " + std::to_string(kind) + "\n",
		           "mfma_probe.hip", "mfma_probe_meta.cpp", "mfma probe", p->b)) return 1;
		if (dev != nullptr) p->dev = dev->dev;
		*out = p.release();
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
void x17p_mfma_probe_free(X17pMfmaProbe *p) { delete p; }
int x17p_mfma_probe_launch(X17pMfmaProbe *p, X17hTensor *operands, X17hTensor *out, size_t iterations, double *ops) {
	if (!p->b.kernel) return fail("mfma probe was built without a device");
	size_t const blocks = meta(p->b, "BLOCKS");
	if (operands->t->bytes < 12 * 512 * 16) return fail("mfma probe needs 98304 bytes of operand data");
	if (out->t->bytes < blocks * 512 * 4) return fail("mfma probe needs an output of 4 bytes per thread");
	if (iterations > 0xFFFFFFFFull) return fail("mfma probe: too many iterations");
	void *src = operands->t->ptr, *dst = out->t->ptr;
	size_t n = iterations;
	void *args[3] = {&src, &n, &dst};
	size_t grid[3] = {blocks, 1, 1}, block[3] = {512, 1, 1};
	if (ops != nullptr) {
		*ops = double(blocks) * 8.0 * double(iterations) * double(meta(p->b, "MFMAS_PER_ITERATION")) * double(meta(p->b, "OPS_PER_MFMA"));
	}
	return from_status(p->b.kernel->launch(*p->dev->stream, grid, block, 0, args));
}

int x17p_valu_probe_ops(void) { return N_VALU_OPS; }
char const *x17p_valu_probe_op_name(int op) { return op >= 0 && op < N_VALU_OPS ? VALU_OPS[op] : ""; }
int x17p_valu_probe_new(X17hDevice *dev, int op, X17pValuProbe **out) {
	try {
		if (op < 0 || op >= N_VALU_OPS) return fail("valu probe: unknown instruction index");
		auto p = std::make_unique<X17pValuProbe>();
		if (!build(dev, "valu_probe-op" + std::to_string(probe_op_code(op)), std::string("// issue probe: ") + VALU_OPS[op] + "\n#define X17_PROBE_OP " + std::to_string(probe_op_code(op)) + "\n",
		           "valu_probe.hip", "valu_probe_meta.cpp", "valu probe", p->b)) return 1;
		if (dev != nullptr) p->dev = dev->dev;
		*out = p.release();
		return 0;
	} catch (std::exception const &e) { return fail(e.what()); }
}
void x17p_valu_probe_free(X17pValuProbe *p) { delete p; }
int x17p_valu_probe_launch(X17pValuProbe *p, X17hTensor *src, X17hTensor *out, size_t waves_per_simd, size_t iterations, double *instructions) {
	if (!p->b.kernel) return fail("valu probe was built without a device");
	if (waves_per_simd == 0 || waves_per_simd > 8) return fail("valu probe: 1 to 8 wavefronts per SIMD");
	size_t const blocks = meta(p->b, "BLOCKS_PER_WAVE_PER_SIMD") * waves_per_simd;
	if (src->t->bytes < 80 * 4) return fail("valu probe needs 80 floats of source data");
	if (out->t->bytes < blocks * 64 * 4) return fail("valu probe needs an output of 4 bytes per thread");
	if (iterations > 0xFFFFFFFFull) return fail("valu probe: too many iterations");
	void *s = src->t->ptr, *d = out->t->ptr;
	size_t n = iterations;
	void *args[3] = {&s, &n, &d};
	size_t grid[3] = {blocks, 1, 1}, block[3] = {64, 1, 1};
	if (instructions != nullptr) *instructions = double(waves_per_simd) * double(iterations) * double(meta(p->b, "INSTRUCTIONS_PER_ITERATION"));
	return from_status(p->b.kernel->launch(*p->dev->stream, grid, block, 0, args));
}

} // extern "C"
