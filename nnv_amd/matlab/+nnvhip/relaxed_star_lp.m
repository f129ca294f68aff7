function h = relaxed_star_lp(hin, method, relaxFactor, lp_solver, dis_opt)
    % relaxFactor < 1 branches of PosLin.reach_relaxed_star_{range,area,bound,ub,random,static}
    % (PosLin.m:863-1650) on a device set: estimateRanges, the step itself and the row gathers run on
    % the GPU; the n1 = round((1-relaxFactor)*numel(map2)) LPs go to NNV's own lpsolver, fed with the
    % rows of V they need (nnvhip_mex('fetch_rows')) and the set's C, d and predicate bounds.
    % hin: uint64 device handle; h: handle of the output set.
    [lb, ub] = nnvhip_mex('estimate_ranges', hin);
    map1 = find(ub <= 0);
    map2 = find(lb < 0 & ub > 0);
    N  = numel(map2);
    n1 = round((1 - relaxFactor)*N);
    [C, d] = nnvhip_mex('fetch_constraints', hin);
    [plb, pub] = nnvhip_mex('fetch_pred', hin);
    typeA = true;
    switch char(method)
        case 'relax-star-range'                                         % PosLin.m:934-936
            [~, midx] = sort(ub(map2) - lb(map2), 'descend');
            map21 = map2(midx(1:n1)); map22 = map2(midx(n1+1:N));
        case 'relax-star-area'                                          % PosLin.m:1049-1052
            [~, midx] = sort(0.5*(abs(ub(map2)).*abs(lb(map2))), 'descend');
            map21 = map2(midx(1:n1)); map22 = map2(midx(n1+1:N));
        case 'relax-star-random'                                        % PosLin.m:1488-1492
            midx = randperm(N, n1)';
            map21 = map2(midx); map22 = setdiff(map2, map21, 'stable');
        case 'relax-star-static'                                        % PosLin.m:1604-1605
            map21 = map2(1:n1); map22 = map2(n1+1:N);
        case 'relax-star-bound'                                         % PosLin.m:1167-1176
            typeA = false;
            [~, midx] = sort([ub(map2); abs(lb(map2))], 'descend');
            midx1 = midx(1:2*n1);
            map21 = map2(midx1(midx1 <= N)); map22 = map2(midx1(midx1 > N) - N);
        case 'relax-star-ub'                                            % PosLin.m:1326-1338
            typeA = false;
            [~, midx_u] = sort(ub(map2), 'descend');
            [~, midx_l] = sort(abs(lb(map2)), 'descend');
            if 2*n1 <= N
                map21 = map2(midx_u(1:2*n1)); map22 = [];
            else
                map21 = map2(midx_u(1:N)); map22 = map2(midx_l(1:2*n1 - N));
            end
        otherwise
            error('This reachability method does not exist');
    end
    xmax = extremes(hin, map21, -1, C, d, plb, pub, lp_solver);         % Star.getMaxs, Star.m:898-970
    map4 = map21(xmax <= 0);
    map11 = [map1; map4(:)];
    map6 = map21(xmax > 0);
    if typeA
        xmin = extremes(hin, map6, 1, C, d, plb, pub, lp_solver);       % Star.getMins, Star.m:784-856
        keep = xmin < 0;
        xmax1 = xmax(xmax > 0);
        index = [map22(:); map6(keep)];                                 % map9
        lbs = [lb(map22); xmin(keep)];
        ubs = [ub(map22); xmax1(keep)];
    else
        ub(map6) = xmax(xmax > 0);
        map23 = setdiff(map22, map4, 'stable');
        xmin = extremes(hin, map23, 1, C, d, plb, pub, lp_solver);
        lb(map23(xmin < 0)) = xmin(xmin < 0);
        index = setdiff(setdiff(map2, map4, 'stable'), map23(xmin >= 0), 'stable');   % map24
        lbs = lb(index); ubs = ub(index);
    end
    if strcmp(dis_opt, 'display')
        fprintf('\n(%d+%d =%d)/%d neurons have ub <= 0', numel(map1), numel(map4), numel(map11), numel(ub));
        fprintf('\nConstruct new star set, %d new predicate variables are introduced', numel(index));
    end
    h = nnvhip_mex('relu_apply_lists', hin, map11, index, lbs, ubs);
end

function x = extremes(hin, map, sgn, C, d, plb, pub, lp_solver)
    % min (sgn = 1) or max (sgn = -1) of the listed states: Star.getMin / getMax, Star.m:744-781, 859-895
    x = zeros(numel(map), 1);
    if isempty(map), return; end
    rows = nnvhip_mex('fetch_rows', hin, map);
    for i = 1:numel(map)
        f = rows(i, 2:end);
        if all(f == 0)
            x(i) = rows(i, 1);
        else
            [fval, exitflag] = lpsolver(sgn*f, C, d, [], [], plb, pub, lp_solver);
            if ~ismember(exitflag, ["l1", "g5"])
                error('Cannot find an optimal solution, exitflag = ' + string(exitflag));
            end
            x(i) = sgn*fval + rows(i, 1);
        end
    end
end
