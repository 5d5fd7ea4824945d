'use strict';
// Flag registry, after tfjs-core/src/environment.ts:31-137 and flags.ts:25-68: flags are
// registered with an evaluation function, evaluated lazily on first get(), and may be
// overridden with set().  Flags can also be given as TFJS_FLAGS="A:1,B:true" in the
// process environment (the reference reads ?tfjsflags= from the page URL).
class Environment {
  constructor() {
    this.flags = {};
    this.flagRegistry = {};
    this.overrides = {};
    const spec = (typeof process !== 'undefined' && process.env && process.env.TFJS_FLAGS) || '';
    spec.split(',').forEach(kv => {
      const parts = kv.split(':');
      if (parts.length === 2) this.overrides[parts[0]] = parseValue(parts[0], parts[1]);
    });
  }
  registerFlag(flagName, evaluationFn, setHook) {
    this.flagRegistry[flagName] = {evaluationFn, setHook};
    if (this.overrides[flagName] != null) this.set(flagName, this.overrides[flagName]);
  }
  get(flagName) {
    if (flagName in this.flags) return this.flags[flagName];
    this.flags[flagName] = this.evaluateFlag(flagName);
    return this.flags[flagName];
  }
  getNumber(flagName) { return this.get(flagName); }
  getBool(flagName) { return this.get(flagName); }
  getFlags() { return this.flags; }
  set(flagName, value) {
    if (this.flagRegistry[flagName] == null) {
      throw new Error(`Cannot set flag ${flagName} as it has not been registered.`);
    }
    this.flags[flagName] = value;
    if (this.flagRegistry[flagName].setHook != null) this.flagRegistry[flagName].setHook(value);
  }
  evaluateFlag(flagName) {
    if (this.flagRegistry[flagName] == null) {
      throw new Error(`Cannot evaluate flag '${flagName}': no evaluation function found.`);
    }
    return this.flagRegistry[flagName].evaluationFn();
  }
  reset() { this.flags = {}; }
}

function parseValue(flagName, value) {
  value = value.toLowerCase();
  if (value === 'true' || value === 'false') return value === 'true';
  if (`${+value}` === value) return +value;
  throw new Error(`Could not parse value flag value ${value} for flag ${flagName}.`);
}

const ENV = new Environment();
ENV.registerFlag('DEBUG', () => false, debugValue => {
  if (debugValue) {
    console.warn('Debugging mode is ON. The output of every math call will be downloaded to ' +
                 'CPU and checked for NaNs. This significantly impacts performance.');
  }
});
ENV.registerFlag('IS_NODE', () => typeof process !== 'undefined' && !!process.versions && !!process.versions.node);
ENV.registerFlag('IS_BROWSER', () => false);
ENV.registerFlag('PROD', () => false);
ENV.registerFlag('IS_TEST', () => false);
// hip backend flags
ENV.registerFlag('HIP_DEVICE', () => 0);
// false = run bias / activation as the reference's separate passes instead of the epilogue
ENV.registerFlag('HIP_FUSE_EPILOGUE', () => true);
// conv2d / depthwiseConv2D / batchMatMul wait for the add(bias) and relu | clip that may follow
ENV.registerFlag('HIP_DEFER_EPILOGUE', () => true);

module.exports = {Environment, ENV};
