// Algorithmic work of one compute operation: the FLOP and byte counts that
// roofline figures are computed from.  Every tensor an operation reads or
// writes is counted once at its dense size; nothing here depends on how a
// kernel is implemented.
#include "ir.h"

namespace dnnc {

const char *op_class(const Op *op) {
  switch (op->kind) {
    case OP_CONVFWD:
    case OP_CONV_BIAS_ACTIV:
    case OP_CONV_BIAS_ADD_ACTIV: return (op->dimB[1] == 1 && op->group > 1) ? "conv_depthwise" : "conv_dense";
    case OP_CONV_BIAS_ACTIV_MAXPOOL: return "conv_dense";
    case OP_CONV_ADD_CONV_ACTIV: return "conv_dense";
    case OP_MATMUL2D: return "gemm";
    case OP_MATMULND:
    case OP_MATMUL_BIAS: return "matmul";
    case OP_SOFTMAX: return "softmax";
    case OP_ATTENTION: return "attention";
    case OP_LAYERNORM: return "layernorm";
    case OP_REDUCE: return "reduce";
    case OP_MAXPOOL:
    case OP_AVGPOOL: return "pool";
    case OP_FLATTEN:
    case OP_RESHAPE:
    case OP_TRANSPOSE:
    case OP_CONCAT:
    case OP_SQUEEZE:
    case OP_UNSQUEEZE:
    case OP_EXPAND:
    case OP_GATHER: return "move";
    default: return "elementwise";
  }
}

void op_work(const Op *op, double &flops, double &bytes) {
  flops = 0;
  bytes = 0;
  const Value *out = op->operands.back();
  const double es = (double)dtype_bytes(out->dtype);
  const double n_out = (double)shape_numel(op->result ? op->result->shape : out->shape);
  auto n_in = [&](size_t i) { return (double)shape_numel(op->operands[i]->shape); };
  switch (op->kind) {
    case OP_CONVFWD:
    case OP_CONV_BIAS_ACTIV:
    case OP_CONV_BIAS_ADD_ACTIV: {
      const double crs = (double)(op->dimB[1] * op->dimB[2] * op->dimB[3]);
      flops = 2.0 * n_out * crs;
      bytes = ((double)shape_numel(op->dimA) + (double)shape_numel(op->dimB) + n_out +
               (op->kind != OP_CONVFWD ? (double)op->dimB[0] : 0.0) +
               (op->kind == OP_CONV_BIAS_ADD_ACTIV ? n_out : 0.0)) * es;
      break;
    }
    case OP_CONV_ADD_CONV_ACTIV: {  // both convolutions' products; every tensor the call touches once
      const double crs = (double)(op->dimB[1] * op->dimB[2] * op->dimB[3]), crs2 = (double)(op->dimB2[1] * op->dimB2[2] * op->dimB2[3]);
      flops = 2.0 * n_out * (crs + crs2);
      bytes = ((double)shape_numel(op->dimA) + (double)shape_numel(op->dimB) + (double)shape_numel(op->dimA2) +
               (double)shape_numel(op->dimB2) + 2.0 * (double)op->dimB[0] + n_out) * es;
      break;
    }
    case OP_CONV_BIAS_ACTIV_MAXPOOL: {  // the convolution's products (its output extents, not the pooled ones); the pooling's compares are not counted
      const Shape &dx = op->dimA, &dw = op->dimB;
      const double P = (double)((dx[2] + 2 * op->pads[0] - dw[2]) / op->strides[0] + 1), Q = (double)((dx[3] + 2 * op->pads[1] - dw[3]) / op->strides[1] + 1);
      flops = 2.0 * (double)dx[0] * (double)dw[0] * P * Q * (double)(dw[1] * dw[2] * dw[3]);
      bytes = ((double)shape_numel(dx) + (double)shape_numel(dw) + (double)dw[0] + n_out) * es;
      break;
    }
    case OP_MATMUL2D: {
      const double k = (double)(op->trans_a ? op->dimA[0] : op->dimA[1]);
      flops = 2.0 * n_out * k;
      bytes = (n_in(0) + n_in(1) + n_out + (op->operands.size() == 4 ? n_in(2) : 0.0)) * es;
      break;
    }
    case OP_MATMULND:
    case OP_MATMUL_BIAS: {
      flops = 2.0 * n_out * (double)op->dimA.back();
      bytes = (n_in(0) + n_in(1) + n_out + (op->kind == OP_MATMUL_BIAS ? n_in(2) : 0.0) +
               (op->kind == OP_MATMUL_BIAS && op->operands.size() == 5 ? n_out : 0.0)) * es;
      break;
    }
    case OP_ATTENTION:  // two products of 2 * B * H * Sq * Sk * D each
      flops = 4.0 * n_out * (double)op->dimB[1];
      bytes = (op->axis ? 4.0 * n_out : n_in(0) + n_in(1) + n_in(2) + n_out) * es;
      break;
    case OP_ADD:
    case OP_MUL:
      flops = n_out;
      bytes = (n_out + (double)shape_numel(op->dimB) + n_out) * es;
      break;
    case OP_GATHER:
      bytes = 2.0 * n_out * es + n_in(1) * 8.0;
      break;
    case OP_PRELU:
      flops = n_out;
      bytes = (2.0 * n_out + n_in(1)) * es;
      break;
    case OP_LAYERNORM:
      flops = 8.0 * n_out;
      bytes = (2.0 * n_out + 2.0 * (double)op->dimA.back()) * es;
      break;
    case OP_SOFTMAX:
      flops = 5.0 * n_out;
      bytes = 2.0 * n_out * es;
      break;
    case OP_REDUCE:
    case OP_MAXPOOL:
    case OP_AVGPOOL:
      flops = (double)shape_numel(op->dimA);
      bytes = ((double)shape_numel(op->dimA) + n_out) * es;
      break;
    case OP_CAST:
      bytes = n_out * (8.0 + es);
      break;
    default:  // unary elementwise and copies: one read, one write
      flops = n_out;
      bytes = 2.0 * n_out * es;
      break;
  }
}

}  // namespace dnnc
