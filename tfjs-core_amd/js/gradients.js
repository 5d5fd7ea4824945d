'use strict';
// tf.grad / tf.grads / tf.valueAndGrad / tf.valueAndGrads / tf.customGrad, after
// tfjs-core/src/gradients.ts:30-388 (same argument checks and messages).
const {ENGINE} = require('./engine');
const {Tensor, Variable} = require('./tensor');
const util = require('./util');
const ops = require('./ops');

const TAPE_OPS = {
  ones: shape => ops.ones(shape),
  zeros: (shape, dtype) => ops.zeros(shape, dtype),
  add: (a, b) => ops.add(a, b)
};

function assertShapesMatch(a, b, prefix) {
  util.assert(util.arraysEqual(a, b), () => prefix + ` Shapes ${a} and ${b} must match`);
}

function checkGrads(grads) {
  if (grads.filter(g => g == null).length > 0) {
    throw new Error(`Cannot compute gradient of y=f(x) with respect to x. Make sure that
    the f you passed encloses all operations that lead from x to y.`);
  }
}

// d f() / d variable for every trainable variable of varList (default: all registered ones),
// keyed by variable name; f must return a scalar (gradients.ts:268-350).
function variableGrads(f, varList) {
  util.assert(typeof f === 'function', () => 'The f passed in variableGrads(f) must be a function');
  util.assert(varList == null || (Array.isArray(varList) && varList.every(v => v instanceof Variable)),
              () => 'The varList passed in variableGrads(f, varList) must be an array of variables');
  const given = varList != null;
  if (!given) varList = Object.keys(ENGINE.registeredVariables).map(n => ENGINE.registeredVariables[n]);
  const frozen = given ? varList.filter(v => !v.trainable) : null;
  const count = varList.length;
  varList = varList.filter(v => v.trainable);
  util.assert(varList.length > 0,
              () => `variableGrads() expects at least one of the input variables to be trainable, ` +
                  `but none of the ${count} variables is trainable.`);
  const {value, grads} = ENGINE.gradients(f, varList, null, true, TAPE_OPS);
  util.assert(grads.some(g => g != null),
              () => 'Cannot find a connection between any variable and the result of the loss ' +
                  'function y=f(x). Please make sure the operations that use variables are inside ' +
                  'the function f passed to minimize().');
  util.assert(value.rank === 0,
              () => `The f passed in variableGrads(f) must return a scalar, but it returned a ` +
                  `rank-${value.rank} tensor`);
  const named = {};
  varList.forEach((v, i) => {
    if (grads[i] != null) named[v.name] = grads[i];
  });
  if (frozen != null) frozen.forEach(v => named[v.name] = null);
  return {value, grads: named};
}

function grad(f) {
  util.assert(typeof f === 'function', () => 'The f passed in grad(f) must be a function');
  return (x, dy) => {
    const $x = ops.convertToTensor(x, 'x', 'tf.grad', null);
    const $dy = dy != null ? ops.convertToTensor(dy, 'dy', 'tf.grad') : null;
    return ENGINE.tidy(() => {
      const {value, grads} = ENGINE.gradients(() => f($x), [$x], $dy, false, TAPE_OPS);
      if ($dy != null) {
        assertShapesMatch(value.shape, $dy.shape,
                          'The shape of dy passed in grad(f)(x, dy) must match the shape returned by f(x)');
      }
      checkGrads(grads);
      return grads[0];
    });
  };
}

function grads(f) {
  util.assert(typeof f === 'function', () => 'The f passed in grads(f) must be a function');
  return (args, dy) => {
    util.assert(Array.isArray(args), () => 'The args passed in grads(f)(args) must be an array ' +
                                           'of `Tensor`s or `TensorLike`s');
    const $args = args.map((a, i) => ops.convertToTensor(a, `args[${i}]`, 'tf.grads', null));
    const $dy = dy != null ? ops.convertToTensor(dy, 'dy', 'tf.grads') : null;
    return ENGINE.tidy(() => {
      const {value, grads} = ENGINE.gradients(() => f.apply(null, $args), $args, $dy, false, TAPE_OPS);
      if ($dy != null) {
        assertShapesMatch(value.shape, $dy.shape,
                          'The shape of dy passed in grads(f)([x1,...], dy) must match the shape returned by f([x1,...])');
      }
      checkGrads(grads);
      return grads;
    });
  };
}

function valueAndGrad(f) {
  util.assert(typeof f === 'function', () => 'The f passed in valueAndGrad(f) must be a function');
  return (x, dy) => {
    util.assert(x instanceof Tensor, () => 'The x passed in valueAndGrad(f)(x) must be a tensor');
    util.assert(dy == null || dy instanceof Tensor,
                () => 'The dy passed in valueAndGrad(f)(x, dy) must be a tensor');
    const {grads, value} = ENGINE.gradients(() => f(x), [x], dy, false, TAPE_OPS);
    checkGrads(grads);
    return {grad: grads[0], value};
  };
}

function valueAndGrads(f) {
  util.assert(typeof f === 'function', () => 'The f passed in valueAndGrads(f) must be a function');
  return (args, dy) => {
    util.assert(Array.isArray(args) && args.every(a => a instanceof Tensor),
                () => 'The args passed in valueAndGrads(f)(args) must be array of tensors');
    util.assert(dy == null || dy instanceof Tensor,
                () => 'The dy passed in valueAndGrads(f)(args, dy) must be a tensor');
    const res = ENGINE.gradients(() => f.apply(null, args), args, dy, false, TAPE_OPS);
    if (dy != null) {
      assertShapesMatch(res.value.shape, dy.shape,
                        'The shape of dy passed in valueAndGrads(f)([x1,...], dy) must match the shape returned by f([x1,...])');
    }
    checkGrads(res.grads);
    return res;
  };
}

function customGrad(f) {
  return ENGINE.customGrad(f);
}

module.exports = {grad, grads, valueAndGrad, valueAndGrads, customGrad, variableGrads};
