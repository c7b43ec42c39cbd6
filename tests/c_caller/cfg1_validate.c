/* A C99 caller of the C-ABI: builds the cfg1 convolution descriptor (1x32x32x16 -> 16 channels, 3x3, stride 1,
 * pad 1) with the library's own parameter generators, validates it on a device-less executor and checks the
 * error path. Compiled by the tests with `gcc -std=c99 -pedantic-errors` against include/ and linked with
 * libnce_hip.so: field order and types of every struct are what the headers say, or this does not work. */
#include <stdio.h>
#include <string.h>

#include "nce_hip.h"
#include "nce_hwtest.h"
#include "nce_params.h"
#include "nce_vpuip.h"

#define CHECK(cond)                                                    \
    do {                                                               \
        if (!(cond)) {                                                 \
            fprintf(stderr, "line %d: %s failed\n", __LINE__, #cond); \
            return 1;                                                  \
        }                                                              \
    } while (0)

static unsigned char in_buf[32 * 32 * 16], out_buf[32 * 32 * 16];
static signed char w_buf[16 * 3 * 3 * 16];

int main(void) {
    uint32_t major = 99, minor = 99;
    nce_executor_desc_t ed;
    nce_executor_handle_t ex = NULL;
    nce_log_handle_t log = NULL;
    nce_cluster_task_desc_t t;
    nce_dpu_task_t v;
    nce_ppe_task_t ppe;
    nce_quant_t out_q;
    int32_t table[16 * 4];
    double w_scale = 0.004;
    int64_t set_bytes = 0, pad_bytes = 0;
    size_t n = 0;
    char text[2048];
    int i;

    CHECK(nceGetVersion(&major, &minor) == NCE_RESULT_SUCCESS && major == NCE_HIP_VERSION_MAJOR && minor == NCE_HIP_VERSION_MINOR);
    ed.device_id = -1; /* no GPU needed: this executor validates only */
    ed.log_level = 2;
    CHECK(nceExecutorCreate(ed, &ex, &log) == NCE_RESULT_SUCCESS && ex != NULL && log != NULL);

    /* weights table and PPE attributes from quantization parameters */
    CHECK(nceConvWeightSetBytes(16, 3, 3, &set_bytes, &pad_bytes) == NCE_RESULT_SUCCESS && set_bytes == 144 && pad_bytes == 0);
    CHECK(nceWeightsTableFill(NCE_ARCH_VPUX37XX, 16, 0, (int32_t)set_bytes, 0xFFFFFF, 0.02, 0.05, &w_scale, 1, NULL, table) == NCE_RESULT_SUCCESS);
    CHECK(nceWeightsTableCheck(table, 16, (int32_t)set_bytes) == NCE_RESULT_SUCCESS);
    CHECK(table[4 * 5 + 0] == 5 * 144 && table[4 * 5 + 1] == 0xFFFFFF);
    out_q.scale = 0.05;
    out_q.zero_point = 128;
    out_q.dtype = NCE_DT_U8;
    CHECK(ncePpeFromPostOp(NCE_ARCH_VPUX37XX, NCE_POSTOP_RELU, 0.0, 0.0, out_q, &ppe) == NCE_RESULT_SUCCESS);
    CHECK(ppe.mode == NCE_PPE_NOOP && ppe.clamp_low == 128 && ppe.clamp_high == 255 && ppe.clamp_domain == NCE_CLAMP_POST_ZP);
    CHECK(ncePpeFuseClamp(out_q, 0.0, 3.0, &ppe) == NCE_RESULT_SUCCESS && ppe.clamp_low == 128 && ppe.clamp_high == 188);

    memset(&t, 0, sizeof(t));
    t.task_type = NCE_TASK_CONV;
    t.input.data = in_buf;
    t.input.dtype = NCE_DT_U8;
    t.input.zero_point = 128;
    t.input.dims[0] = 1, t.input.dims[1] = 16, t.input.dims[2] = 32, t.input.dims[3] = 32;
    t.input.strides_bytes[0] = 32 * 32 * 16, t.input.strides_bytes[1] = 1, t.input.strides_bytes[2] = 32 * 16, t.input.strides_bytes[3] = 16;
    t.output = t.input;
    t.output.data = out_buf;
    t.weights.data = w_buf;
    t.weights.dtype = NCE_DT_I8;
    t.weights.dims[0] = 16, t.weights.dims[1] = 16, t.weights.dims[2] = 3, t.weights.dims[3] = 3;
    t.weights.strides_bytes[0] = 144, t.weights.strides_bytes[1] = 1, t.weights.strides_bytes[2] = 48, t.weights.strides_bytes[3] = 16;
    t.weight_table.data = table;
    t.weight_table.dtype = NCE_DT_SI32;
    t.weight_table.dims[0] = 16, t.weight_table.dims[1] = 1, t.weight_table.dims[2] = 1, t.weight_table.dims[3] = 4;
    t.weight_table.strides_bytes[0] = 16, t.weight_table.strides_bytes[1] = 4, t.weight_table.strides_bytes[2] = 4, t.weight_table.strides_bytes[3] = 4;
    t.kernel_size[0] = t.kernel_size[1] = 3;
    t.kernel_strides[0] = t.kernel_strides[1] = 1;
    t.kernel_pad_left = t.kernel_pad_right = t.kernel_pad_top = t.kernel_pad_bottom = 1;
    memset(&v, 0, sizeof(v));
    v.out_end[0] = 31, v.out_end[1] = 31, v.out_end[2] = 15;
    v.pad_left = v.pad_right = v.pad_top = v.pad_bottom = 1;
    v.mpe_mode = NCE_MPE_CUBOID_16x16;
    t.variants = &v;
    t.num_variants = 1;
    t.ppe = &ppe;
    CHECK(nceClusterTaskValidate(ex, &t) == NCE_RESULT_SUCCESS);

    /* a device-less executor cannot launch, and says so */
    CHECK(nceClusterTaskEnqueue(ex, &t, NULL) == NCE_RESULT_ERROR_UNSUPPORTED);
    /* a wrong field is named in the log (two-call retrieval) */
    t.kernel_size[1] = 12;
    CHECK(nceClusterTaskValidate(ex, &t) == NCE_RESULT_ERROR_INVALID_ARGUMENT);
    CHECK(nceLogHandleGetString(log, &n, NULL) == NCE_RESULT_SUCCESS && n > 1 && n < sizeof(text));
    CHECK(nceLogHandleGetString(log, &n, text) == NCE_RESULT_SUCCESS);
    CHECK(strstr(text, "kernel width") != NULL);
    for (i = 0; i < 3; ++i) CHECK(v.out_start[i] == 0);
    CHECK(nceClusterTaskValidate(NULL, &t) == NCE_RESULT_ERROR_INVALID_NULL_HANDLE);
    CHECK(nceExecutorDestroy(ex) == NCE_RESULT_SUCCESS);
    printf("ok\n");
    return 0;
}
