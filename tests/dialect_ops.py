"""
Small ops written in RETURNN's native-op source dialect (the vocabulary of returnn/native_op.cpp as the op classes of
returnn/native_op.py use it), for testing the HIP op loader.  Each exercises a different part of the vocabulary and has a
few-line numpy restatement in tests/test_gpu_op_loader.py.  They are test material, not part of the package.
"""

from __future__ import annotations


class ElmanScan:
    """
    h_t = tanh(x_t + h_{t-1} W) where the mask is 1, h_{t-1} where it is 0; frames start, start+step, ... as NativeLstm2
    counts them.  Exercises: host int32 scalars, device_malloc/free, Ndarray_memcpy, data_ptr, affine_raw (rocBLAS),
    start_dev_kernel with the default launch shape, assert_cmp, HANDLE_LAST_ERROR; with its gradient code: the derivation
    of the gradient op (grad_input_map as a callable that drops X and hT, bw_out_var giving DX its shape from Y,
    disconnected inputs) and affine_raw with transposed operands.
    """

    in_info = (
        # the gradient op does not take X (see grad_input_map): DX gets its shape from Y, input 5 of the gradient op
        {"name": "X", "ndim": 3, "shape": (None, None, None), "need_contiguous": True, "bw_out_var": {"shape": ((5, 0), (5, 1), (5, 2))}},
        {"name": "W", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "h0", "ndim": 2, "shape": (None, None), "need_contiguous": True},
        {"name": "i", "ndim": 2, "shape": (None, None), "need_contiguous": True, "gradient": "disconnected"},
        {"name": "start", "ndim": 0, "shape": (), "dtype": "int32", "host_memory": True, "gradient": "disconnected"},
        {"name": "step", "ndim": 0, "shape": (), "dtype": "int32", "host_memory": True, "gradient": "disconnected"},
    )
    out_info = (
        {"name": "Y", "ndim": 3, "shape": ((0, 0), (0, 1), (0, 2))},
        {"name": "hT", "ndim": 2, "shape": ((2, 0), (2, 1))},
    )
    c_extra_support_code = {
        "10_cell": """
        DEF_KERNEL void elman_cell(long rows, long width, const float* pre, const float* carry, const float* mask_row, float* out) {
          for (long k = threadIdx.x + (long)blockDim.x * blockIdx.x; k < rows * width; k += (long)gridDim.x * blockDim.x) {
            const float keep = mask_row[k / width];
            out[k] = keep * tanhf(pre[k]) + (1.f - keep) * carry[k];
          }
        }
        """,
        "20_cell_grad": """
        DEF_KERNEL void elman_cell_grad(long rows, long width, const float* y, const float* dy, const float* carry, const float* mask_row,
                                        float* g, float* passed) {
          for (long k = threadIdx.x + (long)blockDim.x * blockIdx.x; k < rows * width; k += (long)gridDim.x * blockDim.x) {
            const float keep = mask_row[k / width];
            const float total = dy[k] + carry[k];
            g[k] = keep * (1.f - y[k] * y[k]) * total;
            passed[k] = (1.f - keep) * total;
          }
        }
        """,
    }
    c_fw_code = """
        Ndarray* X = inputs[0];
        Ndarray* W = inputs[1];
        Ndarray* h0 = inputs[2];
        Ndarray* mask = inputs[3];
        int first = Ndarray_DEV_DATA_int32_scalar(inputs[4]);
        const int stride = Ndarray_DEV_DATA_int32_scalar(inputs[5]);
        Ndarray* Y = *outputs[0];
        Ndarray* hT = *outputs[1];
        assert_cmp(Ndarray_NDIM(X), ==, 3);
        const long frames = Ndarray_DIMS(X)[0];
        const int rows = (int) Ndarray_DIMS(X)[1], width = (int) Ndarray_DIMS(X)[2];
        assert_cmp(Ndarray_DIMS(W)[0], ==, width);
        assert_cmp(Ndarray_DIMS(W)[1], ==, width);
        assert_cmp(Ndarray_DIMS(h0)[0], ==, rows);
        assert_cmp(Ndarray_DIMS(h0)[1], ==, width);
        assert_cmp(Ndarray_DIMS(mask)[0], ==, frames);
        assert_cmp(Ndarray_DIMS(mask)[1], ==, rows);
        assert_cmp(stride, !=, 0);
        assert_cmp(first, >=, 0);
        assert_cmp(first, <, frames);
        if (stride < 0) first = (int) frames - 1 - first;
        const size_t state_bytes = sizeof(float) * rows * width;
        float* pre = (float*) device_malloc(state_bytes);
        float* carry = (float*) device_malloc(state_bytes);
        Ndarray_memcpy(carry, Ndarray_DEV_DATA(h0), state_bytes);
        for (long t = first; t >= 0 && t < frames; t += stride) {
          Ndarray_memcpy(pre, data_ptr(X, (int) t), state_bytes);
          affine_raw(carry, rows, width, Ndarray_DEV_DATA(W), width, width, pre, rows, width);  // pre += carry . W
          start_dev_kernel(elman_cell, (rows, width, pre, carry, Ndarray_DEV_DATA(mask) + t * rows, data_ptr(Y, (int) t)));
          HANDLE_LAST_ERROR();
          Ndarray_memcpy(carry, data_ptr(Y, (int) t), state_bytes);
        }
        Ndarray_memcpy(Ndarray_DEV_DATA(hT), carry, state_bytes);
        device_free(carry);
        device_free(pre);
    """

    # noinspection PyPep8Naming
    @staticmethod
    def grad_input_map(X, W, h0, i, start, step, Y, hT, DY, DhT):
        del X, hT
        return W, h0, i, start, step, Y, DY, DhT

    c_bw_code = """
        Ndarray* W = inputs[0];
        Ndarray* h0 = inputs[1];
        Ndarray* mask = inputs[2];
        int first = Ndarray_DEV_DATA_int32_scalar(inputs[3]);
        const int stride = Ndarray_DEV_DATA_int32_scalar(inputs[4]);
        Ndarray* Y = inputs[5];
        Ndarray* DY = inputs[6];
        Ndarray* DhT = inputs[7];
        Ndarray* DX = *outputs[0];
        Ndarray* DW = *outputs[1];
        Ndarray* Dh0 = *outputs[2];
        const long frames = Ndarray_DIMS(Y)[0];
        const int rows = (int) Ndarray_DIMS(Y)[1], width = (int) Ndarray_DIMS(Y)[2];
        assert_cmp(Ndarray_DIMS(DX)[0], ==, frames);
        assert_cmp(Ndarray_DIMS(DW)[0], ==, width);
        assert_cmp(Ndarray_DIMS(Dh0)[1], ==, width);
        assert_cmp(stride, !=, 0);
        assert_cmp(first, >=, 0);
        assert_cmp(first, <, frames);
        long visited;
        if (stride > 0) visited = (frames - 1 - first) / stride + 1;
        else { first = (int) frames - 1 - first; visited = first / (-stride) + 1; }
        const size_t state_bytes = sizeof(float) * rows * width;
        float* carry = (float*) device_malloc(state_bytes);   // error arriving from the frames after this one
        float* passed = (float*) device_malloc(state_bytes);  // the part that skips a masked frame
        Ndarray_memcpy(carry, Ndarray_DEV_DATA(DhT), state_bytes);
        for (long k = visited - 1; k >= 0; --k) {
          const long t = first + k * stride;
          float* g = data_ptr(DX, (int) t);
          start_dev_kernel(elman_cell_grad, (rows, width, data_ptr(Y, (int) t), data_ptr(DY, (int) t), carry,
                                             Ndarray_DEV_DATA(mask) + t * rows, g, passed));
          HANDLE_LAST_ERROR();
          float* before = (k == 0) ? Ndarray_DEV_DATA(h0) : data_ptr(Y, (int) (t - stride));
          affine_raw(before, rows, width, g, rows, width, Ndarray_DEV_DATA(DW), width, width, true, false);  // DW += before^T . g
          Ndarray_memcpy(carry, passed, state_bytes);
          affine_raw(g, rows, width, Ndarray_DEV_DATA(W), width, width, carry, rows, width, false, true);    // carry += g . W^T
        }
        Ndarray_memcpy(Ndarray_DEV_DATA(Dh0), carry, state_bytes);
        device_free(passed);
        device_free(carry);
    """
    code_version = (2,)


class RowLogSumExp:
    """
    Per row of a matrix: log(sum(exp(x))) and the index of the largest element (int32 output).  One block per row with a
    shared-memory tree reduction.  Exercises: start_dev_kernel2, DEF_SHARED, the __CUDA_ARCH__ guard around
    __syncthreads that op sources use (without it the reduction is wrong), INF_F, an int32 output.
    """

    in_info = ({"name": "x", "ndim": 2, "shape": (None, None), "need_contiguous": True},)
    out_info = (
        {"name": "lse", "ndim": 1, "shape": ((0, 0),)},
        {"name": "arg", "ndim": 1, "shape": ((0, 0),), "dtype": "int32"},
    )
    c_extra_support_code = {
        "01_sync": """
        DEV_FUNC void block_sync() {
        #ifdef __CUDA_ARCH__
          __syncthreads();
        #endif
        }
        """,
        "02_kernel": """
        DEF_KERNEL void row_lse(long cols, const float* x, float* lse, int* arg) {
          DEF_SHARED(float, shared)
          float* best = shared;                       // [blockDim.x]
          int* where = (int*) (shared + blockDim.x);  // [blockDim.x]
          float* total = shared + 2 * blockDim.x;     // [blockDim.x]
          const float* row = x + blockIdx.x * cols;
          float my_best = -INF_F;
          int my_where = 0;
          for (long c = threadIdx.x; c < cols; c += blockDim.x)
            if (row[c] > my_best) { my_best = row[c]; my_where = (int) c; }
          best[threadIdx.x] = my_best;
          where[threadIdx.x] = my_where;
          block_sync();
          for (unsigned half = blockDim.x / 2; half > 0; half /= 2) {
            if (threadIdx.x < half) {
              const float other = best[threadIdx.x + half];
              const int other_where = where[threadIdx.x + half];
              if (other > best[threadIdx.x] || (other == best[threadIdx.x] && other_where < where[threadIdx.x])) {
                best[threadIdx.x] = other;
                where[threadIdx.x] = other_where;
              }
            }
            block_sync();
          }
          const float top = best[0];
          float my_total = 0.f;
          for (long c = threadIdx.x; c < cols; c += blockDim.x) my_total += expf(row[c] - top);
          total[threadIdx.x] = my_total;
          block_sync();
          for (unsigned half = blockDim.x / 2; half > 0; half /= 2) {
            if (threadIdx.x < half) total[threadIdx.x] += total[threadIdx.x + half];
            block_sync();
          }
          if (threadIdx.x == 0) {
            lse[blockIdx.x] = top + logf(total[0]);
            arg[blockIdx.x] = where[0];
          }
        }
        """,
    }
    c_fw_code = """
        Ndarray* x = inputs[0];
        Ndarray* lse = *outputs[0];
        Ndarray* arg = *outputs[1];
        assert_cmp(Ndarray_NDIM(x), ==, 2);
        const long n_rows = Ndarray_DIMS(x)[0], n_cols = Ndarray_DIMS(x)[1];
        assert_cmp(Ndarray_DIMS(lse)[0], ==, n_rows);
        assert_cmp(Ndarray_dtype_size(arg), ==, 4);
        if (n_cols == 0) { %(fail)s }
        if (n_rows > 0) {
          const unsigned threads = 256;
          start_dev_kernel2(row_lse, (unsigned) n_rows, threads, 3 * threads * sizeof(float),
            (n_cols, Ndarray_DEV_DATA(x), Ndarray_DEV_DATA(lse), Ndarray_DEV_DATA_int32(arg)));
          HANDLE_LAST_ERROR();
        }
    """


class BucketSum:
    """
    acc[idx[k]] += values[k] in place on the caller's accumulator, hits per bucket, and twice the values in a dummy output.
    Exercises: int32 input, elem_atomic_add, want_inplace on an output index, want_inplace="dummy_out", zero-initialised
    outputs, Ndarray_SIZE, CHECK_WITH_MSG.
    """

    in_info = (
        {"name": "acc", "ndim": 1, "shape": (None,), "need_contiguous": True, "want_inplace": 0},
        {"name": "values", "ndim": 1, "shape": (None,), "need_contiguous": True, "want_inplace": "dummy_out"},
        {"name": "idx", "ndim": 1, "shape": (None,), "need_contiguous": True, "dtype": "int32"},
    )
    out_info = (
        {"name": "out", "ndim": 1, "shape": ((0, 0),)},
        {"name": "hits", "ndim": 1, "shape": ((0, 0),)},
    )
    c_extra_support_code = {
        "kernel": """
        DEF_KERNEL void bucket_sum(long count, long buckets, float* values, const int* idx, float* acc, float* hits) {
          for (long k = threadIdx.x + (long)blockDim.x * blockIdx.x; k < count; k += (long)gridDim.x * blockDim.x) {
            const int b = idx[k];
            if (b >= 0 && b < buckets) {
              elem_atomic_add(&acc[b], values[k]);
              elem_atomic_add(&hits[b], 1.0f);
            }
            values[k] *= 2.f;
          }
        }
        """
    }
    c_fw_code = """
        assert(n_inputs == 3);
        assert(n_outputs == 3);
        Ndarray* values = inputs[1];
        Ndarray* idx = inputs[2];
        Ndarray* out = *outputs[0];
        Ndarray* hits = *outputs[1];
        Ndarray* doubled = *outputs[2];
        CHECK_WITH_MSG(Ndarray_SIZE(values) == Ndarray_SIZE(idx), "BucketSum: ", Ndarray_SIZE(values), " values but ", Ndarray_SIZE(idx), " indices");
        assert(Ndarray_DEV_DATA(out) == Ndarray_DEV_DATA(inputs[0]));
        assert(Ndarray_DEV_DATA(doubled) == Ndarray_DEV_DATA(values));
        start_dev_kernel(bucket_sum, (Ndarray_SIZE(values), Ndarray_DIMS(out)[0], Ndarray_DEV_DATA(doubled), Ndarray_DEV_DATA_int32(idx),
                                      Ndarray_DEV_DATA(out), Ndarray_DEV_DATA(hits)));
        HANDLE_LAST_ERROR();
    """


class AffineAll:
    """
    Products over all frames and per frame.  Exercises: affine_global with a transposed operand and with a frame offset,
    affine_y_x, Ndarray_set_zero, Ndarray_memset, Ndarray_sgemm in its column-major form.
    """

    in_info = (
        {"name": "A", "ndim": 3, "shape": (None, None, None), "need_contiguous": True},
        {"name": "B", "ndim": 3, "shape": (None, None, None), "need_contiguous": True},
        {"name": "V", "ndim": 2, "shape": (None, None), "need_contiguous": True},
    )
    out_info = (
        {"name": "AtB", "ndim": 2, "shape": ((0, 2), (1, 2))},  # sum_t A[t]^T B[t]
        {"name": "AtB_shift", "ndim": 2, "shape": ((0, 2), (1, 2))},  # sum_t A[t-1]^T B[t]
        {"name": "AV", "ndim": 3, "shape": ((0, 0), (0, 1), (2, 1))},  # A[t] V
        {"name": "VtV", "ndim": 2, "shape": ((2, 1), (2, 1))},  # V^T V through Ndarray_sgemm
    )
    c_fw_code = """
        Ndarray* A = inputs[0];
        Ndarray* B = inputs[1];
        Ndarray* V = inputs[2];
        Ndarray* AtB = *outputs[0];
        Ndarray* AtB_shift = *outputs[1];
        Ndarray* AV = *outputs[2];
        Ndarray* VtV = *outputs[3];
        Ndarray_memset(Ndarray_DEV_DATA(AtB), 0xff, Ndarray_SIZE(AtB) * sizeof(float));  // NaN pattern, then beta = 0
        affine_global(A, B, AtB, true, false, 0, 0.0f);
        Ndarray_set_zero(AtB_shift);
        affine_global(A, B, AtB_shift, true, false, 1);  // beta = 1 on zeros
        const long frames = Ndarray_DIMS(A)[0];
        for (long t = 0; t < frames; ++t)
          affine_y_x((int) t, A, 0, V, (int) t, AV, false, false, 0.0f);
        const int n = (int) Ndarray_DIMS(V)[0], m = (int) Ndarray_DIMS(V)[1];
        const float one = 1.f, zero = 0.f;
        // row-major V [n,m] is column-major [m,n] with leading dimension m; V^T V in row-major terms is (col-major) V_cm V_cm^T
        Ndarray_sgemm('N', 'T', m, m, n, &one, Ndarray_DEV_DATA(V), m, Ndarray_DEV_DATA(V), m, &zero, Ndarray_DEV_DATA(VtV), m);
    """


ALL_OPS = (ElmanScan, RowLogSumExp, BucketSum, AffineAll)
