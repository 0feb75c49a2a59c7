package neureka.devices.hip;

import neureka.Tensor;
import neureka.autograd.ADAction;
import neureka.backend.api.AutoDiffMode;
import neureka.backend.api.DeviceAlgorithm;
import neureka.backend.api.ExecutionCall;
import neureka.backend.api.Operation;
import neureka.backend.api.Result;
import neureka.backend.api.fun.SuitabilityPredicate;
import neureka.backend.api.template.algorithms.AbstractDeviceAlgorithm;
import neureka.backend.hip.Hip;
import neureka.math.Function;
import neureka.math.args.Arg;
import neureka.math.implementations.FunctionConstant;
import neureka.math.implementations.FunctionInput;
import neureka.math.implementations.FunctionVariable;

import java.util.ArrayList;
import java.util.HashMap;
import java.util.LinkedHashSet;
import java.util.List;
import java.util.Map;
import java.util.Set;

/**
 *  Turns a {@link Function} into programs for nk_fused: the counterpart of
 *  neureka.devices.opencl.utility.CLFunctionCompiler (CLFunctionCompiler.java:27-238), which writes OpenCL source and
 *  compiles it at run time.  Here nothing is compiled: the expression tree is lowered to the postfix op-codes the
 *  library's interpreter kernel evaluates per element (NK_FUSE_LOAD / CONST / FUN / DFUN / BIN), and an expression that
 *  exceeds what one launch takes is cut into stages that hand their results on through temporaries.
 *  The derivative kernels come from a symbolic derivative of the tree taken here: Function.getDerivative, which
 *  CLFunctionCompiler uses (:155-157), throws for every activation but ln (AbstractOperation.java:236-238).
 */
public final class HipFunctionCompiler
{
    // what one launch of nk_fused takes (include/neureka_hip.h: NK_FUSE_MAX_*) and its op-codes
    static final int MAX_SRC = 6, MAX_OPS = 32, MAX_STACK = 8, MAX_CONST = 8, MAX_SAVED = 4;
    static final int LOAD = 0, CONST = 1, FUN = 2, DFUN = 3, BIN = 4;
    static final int ADD = 0, SUB = 1, MUL = 2, DIV = 3, MOD = 4, POW = 5;

    enum Kind { INPUT, CONST, FUN, DFUN, OP, TEMP }

    /** A node of the expression tree: inputs, constants, unary functions (and their derivatives), binary operators,
     *  and, once the planner has cut the tree, the results of earlier stages. */
    static final class Node {
        final Kind kind; final int id; final double value; final Node[] children;
        private Node(Kind kind, int id, double value, Node... children) { this.kind = kind; this.id = id; this.value = value; this.children = children; }
        static Node input(int index) { return new Node(Kind.INPUT, index, 0); }
        static Node temp(int stage)  { return new Node(Kind.TEMP, stage, 0); }
        static Node constant(double v) { return new Node(Kind.CONST, 0, v); }
        static Node fun(int funId, Node arg)  { return new Node(Kind.FUN, funId, 0, arg); }
        static Node dfun(int funId, Node arg) { return new Node(Kind.DFUN, funId, 0, arg); }
        static Node op(int opId, Node a, Node b) { return new Node(Kind.OP, opId, 0, a, b); }
        boolean isConst(double v) { return kind == Kind.CONST && value == v; }
        boolean isLeaf() { return children.length == 0; }
    }

    /** One launch: the program, its constants and where its sources come from ({0, k} = input k, {1, s} = result of stage s). */
    static final class Stage {
        final int[] program; final double[] consts; final int[][] leaves;
        Stage(int[] program, double[] consts, int[][] leaves) { this.program = program; this.consts = consts; this.leaves = leaves; }
    }

    private final HipDevice _device;
    private final Function _function;
    private final String _name;
    private final Node _root;
    private final List<Stage> _forward;
    private final Map<Integer, List<Stage>> _derivatives = new HashMap<>();

    public HipFunctionCompiler( HipDevice device, Function toBeOptimized, String functionName ) {
        _device = device;
        _function = toBeOptimized;
        _name = functionName;
        _root = treeOf( toBeOptimized );
        _forward = plan( _root );
    }

    // ---- Function -> tree --------------------------------------------------------------------------------------------
    static Node treeOf( Function f ) {
        if ( f instanceof FunctionInput ) return Node.input( ((FunctionInput) f).index() );
        if ( f instanceof FunctionConstant ) return Node.constant( ((FunctionConstant) f).value() );
        if ( f instanceof FunctionVariable ) throw new IllegalArgumentException( "An indexer ('I[j]') cannot be fused into an elementwise kernel." );
        String id = f.getOperation().getIdentifier();
        List<Function> subs = f.getSubFunctions();
        int funId = Hip.FUN_IDS.indexOf( id );
        if ( funId >= 0 && subs.size() == 1 ) return Node.fun( funId, treeOf( subs.get( 0 ) ) );
        int opId = Hip.OP_IDS.indexOf( id );
        if ( opId < 0 || subs.size() < 2 )
            throw new IllegalArgumentException( "Operation '" + id + "' cannot be fused into an elementwise kernel." );
        Node acc = treeOf( subs.get( 0 ) );                       // a + b + c is one node with three children: folded to the left
        for ( int i = 1; i < subs.size(); i++ ) acc = Node.op( opId, acc, treeOf( subs.get( i ) ) );
        return acc;
    }

    // ---- symbolic derivative, 0 and 1 folded away --------------------------------------------------------------------------
    private static Node mul( Node a, Node b ) {
        if ( a.isConst( 0 ) || b.isConst( 0 ) ) return Node.constant( 0 );
        if ( a.isConst( 1 ) ) return b;
        if ( b.isConst( 1 ) ) return a;
        return Node.op( MUL, a, b );
    }
    private static Node add( Node a, Node b ) { return a.isConst( 0 ) ? b : b.isConst( 0 ) ? a : Node.op( ADD, a, b ); }
    private static Node sub( Node a, Node b ) {
        if ( b.isConst( 0 ) ) return a;
        if ( a.isConst( 0 ) ) return mul( Node.constant( -1 ), b );
        return Node.op( SUB, a, b );
    }
    /** d n / d I[index]; DFUN nodes stand for the derivative of a unary function at its argument. */
    static Node derivativeOf( Node n, int index ) {
        switch ( n.kind ) {
            case INPUT: return Node.constant( n.id == index ? 1 : 0 );
            case CONST: return Node.constant( 0 );
            case FUN:   return mul( Node.dfun( n.id, n.children[ 0 ] ), derivativeOf( n.children[ 0 ], index ) );
            case OP:    break;
            default:    throw new IllegalArgumentException( "Second derivatives of fused functions are not supported." );
        }
        Node u = n.children[ 0 ], v = n.children[ 1 ];
        Node du = derivativeOf( u, index ), dv = derivativeOf( v, index );
        switch ( n.id ) {
            case ADD: return add( du, dv );
            case SUB: return sub( du, dv );
            case MUL: return add( mul( du, v ), mul( u, dv ) );
            case DIV:                                             // du / v - u * dv / v^2
                return sub( du.isConst( 0 ) ? Node.constant( 0 ) : Node.op( DIV, du, v ),
                            mul( dv, Node.op( DIV, u, Node.op( MUL, v, v ) ) ) );
            case POW: {                                           // v * u^(v-1) * du + u^v * ln(u) * dv
                Node first  = mul( mul( v, Node.op( POW, u, Node.op( SUB, v, Node.constant( 1 ) ) ) ), du );
                Node second = mul( mul( Node.op( POW, u, v ), Node.fun( Hip.FUN_IDS.indexOf( "ln" ), u ) ), dv );
                return add( first, second );
            }
            case MOD: return du;                                  // operator/Modulo.java:183-185: the derivative of the first operand
            default:  throw new IllegalArgumentException( "Operator " + n.id + " has no fused derivative." );
        }
    }

    // ---- what a tree costs one launch ----------------------------------------------------------------------------------------
    private static final class Cost {
        int ops, depth; final Set<Long> leaves = new LinkedHashSet<>(); final Set<Double> consts = new LinkedHashSet<>();
    }
    private static long leafKey( Node n ) { return ( n.kind == Kind.TEMP ? 1L << 32 : 0L ) | n.id; }
    private static Cost cost( Node n ) {
        Cost c = new Cost();
        switch ( n.kind ) {
            case INPUT: case TEMP: c.ops = 1; c.depth = 1; c.leaves.add( leafKey( n ) ); return c;
            case CONST:            c.ops = 1; c.depth = 1; c.consts.add( n.value ); return c;
            case FUN: case DFUN: {
                Cost a = cost( n.children[ 0 ] );
                a.ops += 1;
                return a;
            }
            default: {
                Cost a = cost( n.children[ 0 ] ), b = cost( n.children[ 1 ] );
                c.ops = a.ops + b.ops + 1;
                c.depth = Math.max( a.depth, b.depth + 1 );
                c.leaves.addAll( a.leaves ); c.leaves.addAll( b.leaves );
                c.consts.addAll( a.consts ); c.consts.addAll( b.consts );
                return c;
            }
        }
    }
    /** How many computed operands wait at once for the evaluation of their right-hand neighbour: the kernel works on one
     *  accumulator, reads plain sources and constants where they are used, and saves a computed operand that has to wait. */
    private static int saved( Node root ) {
        final int LAZY = 0, ACC = 1, SAVED = 2;
        final List<Integer> stack = new ArrayList<>();
        final int[] state = { 0, 0 };                             // saved now, peak
        Runnable saveAcc = () -> {
            for ( int i = 0; i < stack.size(); i++ ) if ( stack.get( i ) == ACC ) { stack.set( i, SAVED ); state[ 0 ]++; }
            state[ 1 ] = Math.max( state[ 1 ], state[ 0 ] );
        };
        new Object() {
            void walk( Node m ) {
                if ( m.isLeaf() ) { stack.add( LAZY ); return; }
                if ( m.kind == Kind.FUN || m.kind == Kind.DFUN ) {
                    walk( m.children[ 0 ] );
                    if ( stack.get( stack.size() - 1 ) == LAZY ) { saveAcc.run(); stack.set( stack.size() - 1, ACC ); }
                    return;
                }
                walk( m.children[ 0 ] ); walk( m.children[ 1 ] );
                int rhs = stack.remove( stack.size() - 1 ), lhs = stack.remove( stack.size() - 1 );
                if ( lhs == LAZY && rhs == LAZY ) saveAcc.run();
                else if ( lhs == SAVED ) state[ 0 ]--;
                stack.add( ACC );
            }
        }.walk( root );
        return state[ 1 ];
    }
    private static boolean fits( Node n ) {
        Cost c = cost( n );
        return c.ops <= MAX_OPS && c.depth <= MAX_STACK && c.leaves.size() <= MAX_SRC && c.consts.size() <= MAX_CONST && saved( n ) <= MAX_SAVED;
    }

    // ---- tree -> stages --------------------------------------------------------------------------------------------------------
    private static Stage lower( Node root ) {
        final List<Long> leaves = new ArrayList<>();
        final List<Double> consts = new ArrayList<>();
        final List<Integer> program = new ArrayList<>();
        new Object() {
            void walk( Node m ) {
                switch ( m.kind ) {
                    case INPUT: case TEMP: {
                        long key = leafKey( m );
                        if ( !leaves.contains( key ) ) leaves.add( key );
                        program.add( LOAD ); program.add( leaves.indexOf( key ) );
                        return;
                    }
                    case CONST:
                        if ( !consts.contains( m.value ) ) consts.add( m.value );
                        program.add( CONST ); program.add( consts.indexOf( m.value ) );
                        return;
                    case FUN: case DFUN:
                        walk( m.children[ 0 ] );
                        program.add( m.kind == Kind.FUN ? FUN : DFUN ); program.add( m.id );
                        return;
                    default:
                        walk( m.children[ 0 ] ); walk( m.children[ 1 ] );
                        program.add( BIN ); program.add( m.id );
                }
            }
        }.walk( root );
        int[][] where = new int[ leaves.size() ][];
        for ( int i = 0; i < where.length; i++ ) where[ i ] = new int[]{ (int) ( leaves.get( i ) >> 32 ), (int) (long) leaves.get( i ) };
        return new Stage( program.stream().mapToInt( Integer::intValue ).toArray(), consts.stream().mapToDouble( Double::doubleValue ).toArray(), where );
    }

    /** Cuts an expression that is too large for one launch into stages: the largest sub-expressions are evaluated into
     *  temporaries first, which later stages read as sources.  Every intermediate of a fused program is rounded to the
     *  tensor's element type as the unfused kernels round it, so a temporary holds exactly what the single program would
     *  have had on its stack.  The last stage writes the result. */
    static List<Stage> plan( Node root ) {
        final List<Stage> stages = new ArrayList<>();
        Node last = new Object() {
            Node reduce( Node n ) {
                if ( n.isLeaf() ) return n;
                Node[] children = new Node[ n.children.length ];
                for ( int i = 0; i < children.length; i++ ) children[ i ] = reduce( n.children[ i ] );     // every child fits one launch by itself now
                Node m = new Node( n.kind, n.id, n.value, children );
                while ( !fits( m ) ) {
                    int big = -1;
                    for ( int i = 0; i < children.length; i++ )
                        if ( !children[ i ].isLeaf() && ( big < 0 || cost( children[ i ] ).ops > cost( children[ big ] ).ops ) ) big = i;
                    stages.add( lower( children[ big ] ) );
                    children[ big ] = Node.temp( stages.size() - 1 );
                    m = new Node( n.kind, n.id, n.value, children );
                }
                return m;
            }
        }.reduce( root );
        stages.add( lower( last ) );
        return stages;
    }

    // ---- the operation: CLFunctionCompiler.optimize (CLFunctionCompiler.java:48-98) ---------------------------------------------
    public Operation optimize() {
        int numberOfArgs = _function.numberOfArgs();
        return Operation
                .builder()
                .identifier( _name )
                .operator( _name )
                .arity( numberOfArgs )
                .isIndexer( false )
                .isOperator( false )
                .isDifferentiable( true )
                .isInline( false )
                .stringifier(
                    children -> {
                        String expression = String.join( ", ", children );
                        if ( expression.charAt( 0 ) == '(' && expression.charAt( expression.length() - 1 ) == ')' )
                            return _name + expression;
                        return _name + "(" + expression + ")";
                    }
                )
                .build()
                .setAlgorithm(
                    DeviceAlgorithm
                        .withName( "generic_algorithm_for_" + _name )
                        .setIsSuitableFor( call -> SuitabilityPredicate.GOOD )
                        .setAutogradModeFor( call -> AutoDiffMode.BACKWARD_ONLY )
                        .setExecution(
                            ( outerCaller, outerCall ) ->
                                Result.of( AbstractDeviceAlgorithm.executeFor(
                                    outerCaller, outerCall,
                                    call -> AbstractDeviceAlgorithm.executeDeviceAlgorithm( call )
                                ) )
                                .withAutoDiff( ( caller, call ) -> ADAction.of( target -> Function.of( caller.toString(), false ).derive( new Tensor[]{ target.error() }, 0 ) ) )
                        )
                        .setCallPreparation(
                            call -> {
                                if ( call.input( 0 ) == null )       // the drain: every element is written by the last stage, so it is
                                    call = call.withInputAt( 0, _device.uninitializedLike( call.input( 1 ) ) );   // neither built on the host nor filled
                                return call;
                            }
                        )
                        .buildFunAlgorithm()
                        .setImplementationFor( HipDevice.class, this::_fusedKernelsFor )
                );
    }

    /** CLFunctionCompiler._adHocKernelFor (:101-199): slot 0 is the drain, slot p + 1 holds input p. */
    private Tensor<?> _fusedKernelsFor( ExecutionCall<?> call ) {
        int d = call.getValOf( Arg.DerivIdx.class );
        List<Stage> stages = d < 0 ? _forward : _derivatives.computeIfAbsent( d, i -> plan( derivativeOf( _root, i ) ) );
        Tensor<?> drain = call.input( 0 );
        List<Tensor<Number>> temps = new ArrayList<>();
        try {
            for ( int s = 0; s < stages.size(); s++ ) {
                Stage stage = stages.get( s );
                boolean isLast = s == stages.size() - 1;
                Tensor<?> out = isLast ? drain : _device.uninitializedLike( drain );
                if ( !isLast ) temps.add( (Tensor<Number>) out );
                Tensor<?>[] srcs = new Tensor[ Math.max( 1, stage.leaves.length ) ];
                for ( int k = 0; k < stage.leaves.length; k++ )
                    srcs[ k ] = stage.leaves[ k ][ 0 ] == 0 ? call.input( stage.leaves[ k ][ 1 ] + 1 ) : temps.get( stage.leaves[ k ][ 1 ] );
                if ( stage.leaves.length == 0 ) srcs[ 0 ] = call.input( 1 );     // a constant expression: a source only for the launch's shape
                Hip.fused( _device, stage.program, stage.consts, out, srcs );
            }
        } finally {
            temps.forEach( _device::free );                           // back to the pool; the stream orders the launches that still read them
        }
        return drain;
    }
}
