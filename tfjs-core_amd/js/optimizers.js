'use strict';
// tf.train.*: the optimizers of tfjs-core/src/optimizers/ (sgd_optimizer.ts, momentum_optimizer.ts,
// adagrad_optimizer.ts, adadelta_optimizer.ts, adam_optimizer.ts, adamax_optimizer.ts,
// rmsprop_optimizer.ts, optimizer.ts, optimizer_constructors.ts) over the tape of this host.
//
// One driver does what every reference optimizer repeats: walk the named gradients, create the
// per-variable state ("slots": non-trainable variables named <variable>/<suffix>) on first
// sight, run the update rule inside a tidy and assign the results.  A rule is a table: its
// slots with their initial values, and step(value, gradient, slots, shared) -> {value, slots}.
// Every update is a handful of elementwise kernels on device-resident buffers; nothing is read
// back to the host.
const {ENGINE} = require('./engine');
const ops = require('./ops');
const {variableGrads} = require('./gradients');
const util = require('./util');

const EPSILON_FLOAT32 = 1e-7;  // KernelBackend.epsilon() for 32-bit floats (backends/backend.ts:646-648)

const s = v => ops.scalar(v);

class Optimizer {
  // spec: {name, slots: [{suffix, init: value => Tensor}], step, shared?: {begin, end, create, dispose}}
  constructor(spec) {
    this.spec = spec;
    this.iterations_ = 0;
    this.state = [];  // per variable position: {suffix: {originalName, variable}}
    this.sharedState = spec.createShared ? ENGINE.tidy(() => spec.createShared()) : null;
  }

  get iterations() { return this.iterations_; }

  // Runs f, differentiates it with respect to the trainable variables (varList or all),
  // applies the update and returns the cost when asked to (optimizer.ts:54-72).
  minimize(f, returnCost, varList) {
    const {value, grads} = this.computeGradients(f, varList);
    if (varList != null) {
      this.applyGradients(varList.map(v => ({name: v.name, tensor: grads[v.name]})));
    } else {
      this.applyGradients(grads);
    }
    Object.keys(grads).forEach(name => {
      if (grads[name] != null) grads[name].dispose();
    });
    if (returnCost) return value;
    value.dispose();
    return null;
  }

  computeGradients(f, varList) { return variableGrads(f, varList); }

  // variableGradients: {name: Tensor} or [{name, tensor}]
  applyGradients(variableGradients) {
    const listed = Array.isArray(variableGradients);
    const names = listed ? variableGradients.map(v => v.name) : Object.keys(variableGradients);
    ENGINE.tidy(() => {
      const shared = this.spec.begin ? this.spec.begin(this.sharedState) : null;
      names.forEach((name, i) => {
        const value = ENGINE.registeredVariables[name];
        if (this.state[i] == null) {
          this.state[i] = {};
          this.spec.slots.forEach(slot => {
            this.state[i][slot.suffix] = {
              originalName: `${name}/${slot.suffix}`,
              variable: ENGINE.tidy(() => slot.init(value).variable(false))
            };
          });
        }
        const gradient = listed ? variableGradients[i].tensor : variableGradients[name];
        if (gradient == null) return;
        const slots = {};
        Object.keys(this.state[i]).forEach(k => slots[k] = this.state[i][k].variable);
        ENGINE.tidy(() => {
          const next = this.spec.step(value, gradient, slots, shared);
          Object.keys(next.slots || {}).forEach(k => slots[k].assign(next.slots[k]));
          value.assign(next.value);
        });
      });
      if (this.spec.end) this.spec.end(this.sharedState);
    });
    this.iterations_++;
  }

  // The slot variables in creation order, as {name, tensor} (optimizer.ts getWeights of the
  // subclasses, without the iteration counter).
  getSlotVariables() {
    const out = [];
    this.spec.slots.forEach(slot => this.state.forEach(st => {
      if (st != null) out.push({name: st[slot.suffix].originalName, tensor: st[slot.suffix].variable});
    }));
    return out;
  }

  dispose() {
    this.state.forEach(st => {
      if (st != null) Object.keys(st).forEach(k => st[k].variable.dispose());
    });
    this.state = [];
    if (this.sharedState != null) {
      Object.keys(this.sharedState).forEach(k => this.sharedState[k].dispose());
      this.sharedState = null;
    }
  }
}

const zerosOf = value => ops.zerosLike(value);

// value <- value - lr * g  (sgd_optimizer.ts:41-58)
function sgd(learningRate) {
  return new Optimizer({
    name: 'SGD', slots: [],
    step: (value, g) => ({value: ops.add(ops.mul(s(-learningRate), g), value)})
  });
}

// acc <- m * acc + g;  value <- value - lr * acc   (Nesterov: value - lr * (g + m * acc))
// (momentum_optimizer.ts:48-86)
function momentum(learningRate, momentumValue, useNesterov) {
  return new Optimizer({
    name: 'Momentum', slots: [{suffix: 'momentum', init: zerosOf}],
    step: (value, g, st) => {
      const acc = ops.add(ops.mul(s(momentumValue), st.momentum), g);
      const dir = useNesterov ? ops.add(g, ops.mul(acc, s(momentumValue))) : acc;
      return {value: ops.add(ops.mul(s(-learningRate), dir), value), slots: {momentum: acc}};
    }
  });
}

// acc <- acc + g^2;  value <- value - lr * g / sqrt(acc + eps)  (adagrad_optimizer.ts:44-82)
function adagrad(learningRate, initialAccumulatorValue) {
  if (initialAccumulatorValue == null) initialAccumulatorValue = 0.1;
  return new Optimizer({
    name: 'Adagrad',
    slots: [{suffix: 'accumulator', init: v => ops.fill(v.shape, initialAccumulatorValue)}],
    step: (value, g, st) => {
      const acc = ops.add(st.accumulator, ops.square(g));
      const update = ops.mul(ops.div(g, ops.sqrt(ops.add(acc, s(EPSILON_FLOAT32)))), s(-learningRate));
      return {value: ops.add(update, value), slots: {accumulator: acc}};
    }
  });
}

// (adadelta_optimizer.ts:51-103)
function adadelta(learningRate, rho, epsilon) {
  if (learningRate == null) learningRate = 0.001;
  if (rho == null) rho = 0.95;
  if (epsilon == null) epsilon = EPSILON_FLOAT32;
  return new Optimizer({
    name: 'Adadelta',
    slots: [{suffix: 'accum_grad', init: zerosOf}, {suffix: 'accum_var', init: zerosOf}],
    step: (value, g, st) => {
      const accGrad = ops.add(ops.mul(st.accum_grad, s(rho)), ops.mul(ops.square(g), s(1 - rho)));
      const updates = ops.mul(ops.div(ops.sqrt(ops.add(st.accum_var, s(epsilon))),
                                      ops.sqrt(ops.add(st.accum_grad, s(epsilon)))), g);
      const accVar = ops.add(ops.mul(st.accum_var, s(rho)), ops.mul(ops.square(updates), s(1 - rho)));
      return {value: ops.add(ops.mul(updates, s(-learningRate)), value),
              slots: {accum_grad: accGrad, accum_var: accVar}};
    }
  });
}

// (adam_optimizer.ts:41-113): the running powers of beta1 and beta2 are variables of the
// optimizer, advanced once per applyGradients.
function adam(learningRate, beta1, beta2, epsilon) {
  if (learningRate == null) learningRate = 0.001;
  if (beta1 == null) beta1 = 0.9;
  if (beta2 == null) beta2 = 0.999;
  if (epsilon == null) epsilon = EPSILON_FLOAT32;
  return new Optimizer({
    name: 'Adam',
    slots: [{suffix: 'm', init: zerosOf}, {suffix: 'v', init: zerosOf}],
    createShared: () => ({accBeta1: s(beta1).variable(), accBeta2: s(beta2).variable()}),
    begin: sh => ({c1: ops.sub(s(1), sh.accBeta1), c2: ops.sub(s(1), sh.accBeta2)}),
    step: (value, g, st, sh) => {
      const m = ops.add(ops.mul(st.m, s(beta1)), ops.mul(g, s(1 - beta1)));
      const v = ops.add(ops.mul(st.v, s(beta2)), ops.mul(ops.square(g), s(1 - beta2)));
      const mHat = ops.div(m, sh.c1), vHat = ops.div(v, sh.c2);
      const update = ops.mul(ops.div(mHat, ops.add(ops.sqrt(vHat), s(epsilon))), s(-learningRate));
      return {value: ops.add(update, value), slots: {m, v}};
    },
    end: sh => {
      sh.accBeta1.assign(ops.mul(sh.accBeta1, s(beta1)));
      sh.accBeta2.assign(ops.mul(sh.accBeta2, s(beta2)));
    }
  });
}

// (adamax_optimizer.ts:44-117)
function adamax(learningRate, beta1, beta2, epsilon, decay) {
  if (learningRate == null) learningRate = 0.002;
  if (beta1 == null) beta1 = 0.9;
  if (beta2 == null) beta2 = 0.999;
  if (epsilon == null) epsilon = EPSILON_FLOAT32;
  if (decay == null) decay = 0.0;
  return new Optimizer({
    name: 'Adamax',
    slots: [{suffix: 'm', init: zerosOf}, {suffix: 'v', init: zerosOf}],
    createShared: () => ({iteration: s(0).variable(), accBeta1: s(beta1).variable()}),
    begin: sh => ({
      c1: ops.sub(s(1), sh.accBeta1),
      lr: ops.div(s(-learningRate), ops.add(ops.mul(sh.iteration, s(decay)), s(1)))
    }),
    step: (value, g, st, sh) => {
      const m = ops.add(ops.mul(st.m, s(beta1)), ops.mul(g, s(1 - beta1)));
      const v = ops.maximum(ops.mul(st.v, s(beta2)), ops.abs(g));
      const update = ops.mul(ops.div(sh.lr, sh.c1), ops.div(m, ops.add(v, s(epsilon))));
      return {value: ops.add(update, value), slots: {m, v}};
    },
    end: sh => {
      sh.iteration.assign(ops.add(sh.iteration, s(1)));
      sh.accBeta1.assign(ops.mul(sh.accBeta1, s(beta1)));
    }
  });
}

// (rmsprop_optimizer.ts:57-146)
function rmsprop(learningRate, decay, momentumValue, epsilon, centered) {
  if (decay == null) decay = 0.9;
  if (momentumValue == null) momentumValue = 0.0;
  if (epsilon == null) epsilon = EPSILON_FLOAT32;
  const slots = [{suffix: 'rms', init: zerosOf}, {suffix: 'momentum', init: zerosOf}];
  if (centered) slots.push({suffix: 'mg', init: zerosOf});
  return new Optimizer({
    name: 'RMSProp', slots,
    step: (value, g, st) => {
      const rms = ops.add(ops.mul(st.rms, s(decay)), ops.mul(ops.square(g), s(1 - decay)));
      const next = {rms};
      let denom;
      if (centered) {
        const mg = ops.add(ops.mul(st.mg, s(decay)), ops.mul(g, s(1 - decay)));
        next.mg = mg;
        denom = ops.sqrt(ops.sub(rms, ops.add(ops.square(mg), s(epsilon))));
      } else {
        denom = ops.sqrt(ops.add(rms, s(epsilon)));
      }
      const mom = ops.add(ops.mul(st.momentum, s(momentumValue)), ops.div(ops.mul(g, s(learningRate)), denom));
      next.momentum = mom;
      return {value: ops.sub(value, mom), slots: next};
    }
  });
}

function required(name, v) {
  util.assert(v != null, () => `${name} requires a learning rate`);
}

// optimizer_constructors.ts:26-278
const train = {
  sgd: lr => (required('tf.train.sgd', lr), sgd(lr)),
  momentum: (lr, m, nesterov) => (required('tf.train.momentum', lr), momentum(lr, m, nesterov)),
  adagrad: (lr, acc) => (required('tf.train.adagrad', lr), adagrad(lr, acc)),
  adadelta, adam, adamax,
  rmsprop: (lr, decay, m, eps, centered) => (required('tf.train.rmsprop', lr), rmsprop(lr, decay, m, eps, centered))
};

module.exports = {Optimizer, train};
