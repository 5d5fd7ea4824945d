'use strict';
// Reverse-mode tape, after tfjs-core/src/tape.ts:41-195.  A node is what runKernel records
// while a tape is on: {id, name, inputs: {name: Tensor}, outputs: [Tensor], saved: [Tensor],
// gradient: dy => {name: () => Tensor}}.  Only ids, shapes and dtypes of inputs / outputs are
// used here (the tensors themselves may already be disposed); saved tensors are kept clones.

// The nodes that lie on a path from one of `xs` to `y`, in tape order, each with its inputs
// reduced to those that depend on an x (tape.ts:41-131).
function getFilteredNodesXToY(tape, xs, y) {
  const fromX = new Set(xs.map(x => x.id));
  const nodeFromX = new Set();
  for (const node of tape) {
    const names = Object.keys(node.inputs);
    if (names.some(n => fromX.has(node.inputs[n].id))) {
      node.outputs.forEach(o => fromX.add(o.id));
      nodeFromX.add(node.id);
    }
  }
  const toY = new Set([y.id]);
  const nodeToY = new Set();
  for (let i = tape.length - 1; i >= 0; i--) {
    const node = tape[i];
    if (node.outputs.some(o => toY.has(o.id))) {
      Object.keys(node.inputs).forEach(n => toY.add(node.inputs[n].id));
      nodeToY.add(node.id);
    }
  }
  const filtered = [];
  for (const node of tape) {
    if (!nodeFromX.has(node.id) || !nodeToY.has(node.id)) continue;
    const pruned = {};
    Object.keys(node.inputs).forEach(n => {
      if (fromX.has(node.inputs[n].id)) pruned[n] = node.inputs[n];
    });
    filtered.push(Object.assign({}, node, {inputs: pruned}));
  }
  return filtered;
}

// Walks the filtered tape backwards; `grads` maps tensor id -> accumulated gradient and
// must hold dy for y on entry (tape.ts:141-195).  `zeros(shape, dtype)` and `add(a, b)` are
// injected to keep this module free of the op layer.
function backpropagateGradients(grads, filteredTape, tidy, zeros, add, arraysEqual) {
  for (let i = filteredTape.length - 1; i >= 0; i--) {
    const node = filteredTape[i];
    const dys = node.outputs.map(o => grads[o.id] != null ? grads[o.id] : zeros(o.shape, o.dtype));
    if (node.gradient == null) {
      throw new Error(`Cannot compute gradient: gradient function not found for ${node.name}.`);
    }
    const inputGradients = node.gradient(node.outputs.length === 1 ? dys[0] : dys);
    for (const inputName in node.inputs) {
      if (!(inputName in inputGradients)) {
        throw new Error(`Cannot backprop through input ${inputName}. ` +
                        `Available gradients found: ${Object.keys(inputGradients)}.`);
      }
      const dx = tidy(() => inputGradients[inputName]());
      if (dx.dtype !== 'float32') {
        throw new Error(`Error in gradient for op ${node.name}. The gradient of input ` +
                        `${inputName} must have 'float32' dtype, but has '${dx.dtype}'`);
      }
      const x = node.inputs[inputName];
      if (!arraysEqual(dx.shape, x.shape)) {
        throw new Error(`Error in gradient for op ${node.name}. The gradient of input ` +
                        `'${inputName}' has shape '${dx.shape}', which does not match ` +
                        `the shape of the input '${x.shape}'`);
      }
      if (grads[x.id] == null) {
        grads[x.id] = dx;
      } else {
        const cur = grads[x.id];
        grads[x.id] = add(cur, dx);
        cur.dispose();
      }
    }
  }
}

module.exports = {getFilteredNodesXToY, backpropagateGradients};
